"""DeepPPOAgent / DeepPPOContinuousAgent: the host side of the reference's GPU training loop
(deep_agents/ppo/ppo.mojo:742-960, 1558-2840; deep_agents/ppo/ppo_continuous.mojo:171-390,
2180-3300) over this library's fused calls.

`train_gpu` keeps the reference's structure -- collect `rollout_len` steps on `n_envs` device
envs, bootstrap + GAE, `num_epochs` epochs of shuffled minibatches, learning-rate and entropy
annealing, KL early stop -- and its seed schedule for sampling and resets.  What differs is where
the work runs: a collection step is one library call (two launches), an epoch is one library
call, and the host reads back only the list of finished episodes and the KL flag, once per
rollout / epoch.  Network sizes, hyper-parameter names and defaults are the reference's.
"""
import torch

from . import checkpoint, ppo
from .model import Linear, LinearReLU, LinearTanh, StochasticActor, seq
from .optimizer import Adam
from .training import Network, Xavier, Kaiming, init_params_small


class TrainingMetrics:
    """Episode returns / lengths in completion order (core/metrics TrainingMetrics of the reference,
    reduced to what the PPO agents record)."""

    def __init__(self, algorithm_name, environment_name):
        self.algorithm_name, self.environment_name = algorithm_name, environment_name
        self.episode_rewards, self.episode_steps = [], []
        self.rollouts, self.total_steps = 0, 0

    def log_episodes(self, rewards, steps):
        self.episode_rewards.extend(rewards)
        self.episode_steps.extend(steps)

    def mean_reward(self, last=100):
        r = self.episode_rewards[-last:]
        return sum(r) / len(r) if r else 0.0


class _PPOAgentBase:
    continuous = False

    def _build(self, ctx, env):
        raise NotImplementedError

    def train_gpu(self, ctx, env, num_episodes, verbose=False, print_every=10, max_rollouts=None,
                  seed=0):
        """Train on device envs of class `env` until `num_episodes` episodes have finished (or
        `max_rollouts` rollouts have run).  Returns TrainingMetrics."""
        if env.OBS_DIM != self.obs_dim:
            raise ValueError("env OBS_DIM %d != agent obs_dim %d" % (env.OBS_DIM, self.obs_dim))
        self._build(ctx, env)
        metrics = TrainingMetrics("Deep PPO (GPU)" + (" continuous" if self.continuous else ""), env.__name__)
        rb, upd = self.rb, self.upd
        N, T = self.n_envs, self.rollout_len
        env.reset_kernel_gpu(ctx, rb.states, seed)
        rb.obs.copy_(rb.states.view(N, env.STATE_SIZE)[:, :env.OBS_DIM].reshape(-1))
        rb.ep_return.zero_(); rb.ep_length.zero_()
        noise_std = float(getattr(self, "obs_noise_std", 0.0)) if self.continuous else 0.0
        if noise_std > 0.0:
            ppo.add_obs_noise(ctx, rb.obs, N, noise_std, 42)      # ppo_continuous.mojo:2557-2564
        desc = rb.descriptor()
        total_steps, completed = 0, 0
        target_steps = self.target_total_steps or num_episodes * 200
        a_lr0, c_lr0, ent0 = self.actor_lr, self.critic_lr, self.entropy_coef
        while completed < num_episodes:
            if max_rollouts is not None and metrics.rollouts >= max_rollouts:
                break
            rb.done_count.zero_()
            # step t of this rollout draws its seeds from the running step count, which grows by N
            # per step: affine in t, so the whole rollout is one call (one launch where fusable)
            if noise_std > 0.0:
                # observation noise sits between the env step and the next policy forward
                # (ppo_continuous.mojo:2705-2713): the steps are issued one by one
                for t in range(T):
                    ts = total_steps + t * N
                    ppo.rollout_step(ctx, desc, t, ts * 2654435761 + t * 7919, ts * 1103515245 + t * 12345,
                                     ts * 1013904223 + t * 2654435761)
                    ppo.add_obs_noise(ctx, rb.obs, N, noise_std, ts * 2654435761 + t * 7919)
            else:
                ppo.rollout_steps(ctx, desc, 0, T,
                                  total_steps * 2654435761, N * 2654435761 + 7919,
                                  total_steps * 1103515245, N * 1103515245 + 12345,
                                  total_steps * 1013904223, N * 1013904223 + 2654435761)
            total_steps += N * T
            # annealing (ppo.mojo:2385-2406)
            progress = min(1.0, total_steps / float(target_steps))
            if self.anneal_lr:
                self.actor.optimizer.lr = a_lr0 * (1.0 - progress)
                self.critic.optimizer.lr = c_lr0 * (1.0 - progress)
            upd.entropy_coef = ent0 * (1.0 - progress) if self.anneal_entropy else ent0
            upd.update(self.num_epochs, seed=seed * 7919 + metrics.rollouts)
            # the only read-back of the rollout: the finished episodes
            cnt = min(int(rb.done_count.item()), rb.done_cap)
            if cnt:
                metrics.log_episodes(rb.done_returns[:cnt].tolist(), rb.done_lengths[:cnt].tolist())
            # auto-checkpoint whenever the episode count passes a multiple of checkpoint_every
            # (ppo.mojo:2228-2255; the parameters only change between rollouts)
            if (self.checkpoint_every > 0 and self.checkpoint_path != ""
                    and (completed + cnt) // self.checkpoint_every > completed // self.checkpoint_every):
                self.save_checkpoint(self.checkpoint_path)
                if verbose:
                    print("  [Checkpoint saved at episode %d ]" % (completed + cnt), flush=True)
            completed += cnt
            metrics.rollouts += 1
            metrics.total_steps = total_steps
            if verbose and metrics.rollouts % print_every == 0:
                print("rollout %d  steps %d  episodes %d  mean return (last 100) %.2f" % (
                    metrics.rollouts, total_steps, completed, metrics.mean_reward()), flush=True)
        if self.continuous:
            self.train_step_count += total_steps   # ppo_continuous.mojo:3328
        return metrics

    def train_gpu_cpu_env(self, ctx, envs, num_episodes, verbose=False, print_every=10, max_rollouts=None,
                          seed=0):
        """Networks on the device, environments on the host (deep_agents/ppo/ppo.mojo:2846-3960,
        ppo_continuous.mojo:977-2170).  `envs` is a list of exactly n_envs objects of the caller with the
        reference's CPU env interface: reset_obs_list() -> observation, and step_obs(action: int) (discrete
        agent, core/env_traits.mojo:163-184) or step_continuous_vec(action: list) (continuous agent,
        :186-222) -> (observation, reward, done).  Per step: one policy launch, the actions to the host,
        the envs stepped one by one in index order, finished envs reset at once, the observations back to
        the device.  The continuous agent hands the envs  clip(action * action_scale + action_bias, -1, 1)
        and stores the raw action, as the reference does.  When the episode target is reached inside a
        rollout, the rollout's remaining steps are still taken (and their episodes logged) and the call
        then returns without an update: the reference tests the target behind its step loop, not inside
        it (ppo.mojo:3290 and :3454-3456, ppo_continuous.mojo likewise).  GAE, normalisation and
        the epochs are those of train_gpu, on the device."""
        if len(envs) != self.n_envs:
            raise ValueError("expected %d environments, got %d" % (self.n_envs, len(envs)))
        N, T = self.n_envs, self.rollout_len
        aw = self.action_dim if self.continuous else 1
        shape = type("HostEnv", (), dict(ENV_ID=-1, STATE_SIZE=self.obs_dim, OBS_DIM=self.obs_dim,
                                         NUM_ACTIONS=0 if self.continuous else self.num_actions,
                                         ACTION_DIM=aw if self.continuous else 0))
        self._build(ctx, shape)
        rb, upd = self.rb, self.upd
        metrics = TrainingMetrics("Deep PPO (GPU+CPU)" + (" continuous" if self.continuous else ""), "CPU Environment")
        obs_host = torch.zeros(N, self.obs_dim, pin_memory=True)
        act_host = torch.zeros(N * aw, pin_memory=True)
        rew_host, done_host = torch.zeros(T * N, pin_memory=True), torch.zeros(T * N, pin_memory=True)
        actions = torch.zeros(N * aw, device=ctx.device)
        for i, e in enumerate(envs):
            obs_host[i] = torch.as_tensor(e.reset_obs_list(), dtype=torch.float32)
        stream = torch.cuda.stream(ctx.stream)       # the copies go where the library enqueues
        with stream:
            rb.obs.copy_(obs_host.reshape(-1))
        ep_return, ep_steps = [0.0] * N, [0] * N
        total_steps, completed = 0, 0
        target_steps = self.target_total_steps or num_episodes * 200
        a_lr0, c_lr0, ent0 = self.actor_lr, self.critic_lr, self.entropy_coef
        scale, bias = getattr(self, "action_scale", 1.0), getattr(self, "action_bias", 0.0)
        while completed < num_episodes:
            if max_rollouts is not None and metrics.rollouts >= max_rollouts:
                break
            for t in range(T):
                ppo.policy_step(ctx, rb, t, total_steps * 2654435761 + t * 7919, actions)
                with stream:
                    act_host.copy_(actions)
                ctx.synchronize()
                a_list = act_host.tolist()
                for i, e in enumerate(envs):
                    if self.continuous:
                        a = [min(1.0, max(-1.0, a_list[i * aw + k] * scale + bias)) for k in range(aw)]
                        nxt, reward, done = e.step_continuous_vec(a)
                    else:
                        nxt, reward, done = e.step_obs(int(a_list[i]))
                    rew_host[t * N + i] = float(reward)
                    done_host[t * N + i] = 1.0 if done else 0.0
                    ep_return[i] += float(reward)
                    ep_steps[i] += 1
                    if done:
                        metrics.log_episodes([ep_return[i]], [ep_steps[i]])
                        completed += 1
                        if (self.checkpoint_every > 0 and self.checkpoint_path != ""
                                and completed % self.checkpoint_every == 0):
                            self.save_checkpoint(self.checkpoint_path)
                        ep_return[i], ep_steps[i] = 0.0, 0
                        nxt = e.reset_obs_list()
                    obs_host[i] = torch.as_tensor(nxt, dtype=torch.float32)
                total_steps += N
                with stream:
                    rb.obs.copy_(obs_host.reshape(-1))
                ctx.synchronize()       # obs_host is rewritten while the envs of the next step run
            if completed >= num_episodes:
                break
            with stream:
                rb.r_rewards.copy_(rew_host)
                rb.r_dones.copy_(done_host)
            progress = min(1.0, total_steps / float(target_steps))
            if self.anneal_lr:
                self.actor.optimizer.lr = a_lr0 * (1.0 - progress)
                self.critic.optimizer.lr = c_lr0 * (1.0 - progress)
            upd.entropy_coef = ent0 * (1.0 - progress) if self.anneal_entropy else ent0
            upd.update(self.num_epochs, seed=seed * 7919 + metrics.rollouts)
            ctx.synchronize()           # the pinned reward / done arrays are rewritten by the next rollout
            metrics.rollouts += 1
            metrics.total_steps = total_steps
            if verbose and metrics.rollouts % print_every == 0:
                print("rollout %d  steps %d  episodes %d  mean return (last 100) %.2f" % (
                    metrics.rollouts, total_steps, completed, metrics.mean_reward()), flush=True)
        metrics.total_steps = total_steps
        if self.continuous:
            self.train_step_count += total_steps
        return metrics

    def evaluate_gpu(self, ctx, env, num_episodes=100, max_steps=1000, verbose=False, stochastic=True,
                     steps_per_readback=32):
        """DeepPPOContinuousAgent.evaluate_gpu (deep_agents/ppo/ppo_continuous.mojo:703-975): run the
        policy on `n_envs` device envs until `num_episodes` episodes have finished or `max_steps`
        steps have been taken; returns the mean return of the first `num_episodes` finished
        episodes (steps in order, envs in index order within a step), 0.0 if none finished.
        Step `s` samples with seed s * 2654435761 (or takes the mean action when `stochastic` is
        false), steps the envs with seed s and re-initialises finished envs with seed s, as there.

        The discrete agent has no GPU evaluation in the reference; here it gets the same loop with
        categorical sampling or, when `stochastic` is false, the greedy action of its CPU
        `evaluate` (ppo.mojo:1487-1556).

        Rewards and done flags are read back every `steps_per_readback` steps instead of every
        step; the steps issued past the last counted episode do not change the result."""
        if env.OBS_DIM != self.obs_dim:
            raise ValueError("env OBS_DIM %d != agent obs_dim %d" % (env.OBS_DIM, self.obs_dim))
        self.build_networks(ctx)
        N, dev = self.n_envs, ctx.device
        aw = env.ACTION_DIM if self.continuous else 1
        states = torch.zeros(N * env.STATE_SIZE, device=dev)
        obs = torch.zeros(N * env.OBS_DIM, device=dev)
        actions = torch.zeros(N * aw, device=dev)
        log_probs = torch.zeros(N, device=dev)
        actor_out = torch.zeros(N * self.actor.model.OUT_DIM, device=dev)
        K = max(1, int(steps_per_readback))
        rewards = torch.zeros(K * N, device=dev)
        dones = torch.zeros(K * N, device=dev)
        env.reset_kernel_gpu(ctx, states, 0)
        obs.copy_(states.view(N, env.STATE_SIZE)[:, :env.OBS_DIM].reshape(-1))
        if verbose:
            print("Running GPU evaluation with", N, "parallel envs...", flush=True)
        current = [0.0] * N
        episode_rewards = []
        step = 0
        while len(episode_rewards) < num_episodes and step < max_steps:
            k = min(K, max_steps - step)
            for j in range(k):
                s = step + j
                self.actor.model.forward_gpu_no_cache_ws(ctx, actor_out, obs, self.actor.params)
                if not stochastic:
                    ppo.greedy_actions(ctx, actor_out, actions, N, self.continuous)
                elif self.continuous:
                    ppo.sample_continuous_actions(ctx, actor_out, actions, log_probs, s * 2654435761)
                else:
                    ppo.sample_actions(ctx, actor_out, actions, log_probs, s * 2654435761)
                env.step_autoreset_kernel_gpu(ctx, states, actions, rewards[j * N:(j + 1) * N],
                                              dones[j * N:(j + 1) * N], obs, s, s)
            ctx.synchronize()
            r_host = rewards[:k * N].view(k, N).tolist()
            d_host = dones[:k * N].view(k, N).tolist()
            for j in range(k):
                rj, dj = r_host[j], d_host[j]
                for i in range(N):
                    current[i] += rj[i]
                    if dj[i] > 0:
                        episode_rewards.append(current[i])
                        current[i] = 0.0
                        if len(episode_rewards) >= num_episodes:
                            break
                step += 1
                if len(episode_rewards) >= num_episodes:
                    break
        if not episode_rewards:
            if verbose:
                print("Warning: No episodes completed!")
            return 0.0
        avg = sum(episode_rewards) / float(len(episode_rewards))
        if verbose:
            print("GPU EVALUATION SUMMARY (%s Actions)" % ("Continuous" if self.continuous else "Discrete"))
            print("Episodes completed:", len(episode_rewards))
            print("Average reward:", avg)
            print("Min reward:", min(episode_rewards))
            print("Max reward:", max(episode_rewards))
        return avg


class DeepPPOAgent(_PPOAgentBase):
    """deep_agents/ppo/ppo.mojo:742-960: actor obs -> hidden (ReLU) -> hidden (ReLU) -> logits,
    critic obs -> hidden (ReLU) -> hidden (ReLU) -> 1, Xavier initialisation, Adam."""

    def __init__(self, obs_dim, num_actions, hidden_dim=64, rollout_len=128, n_envs=1024,
                 gpu_minibatch_size=256, gamma=0.99, gae_lambda=0.95, clip_epsilon=0.2, actor_lr=0.0003,
                 critic_lr=0.001, entropy_coef=0.01, value_loss_coef=0.5, num_epochs=4,
                 normalize_advantages=True, target_kl=0.015, max_grad_norm=0.5, anneal_lr=True,
                 anneal_entropy=False, target_total_steps=0, clip_value=True, norm_adv_per_minibatch=True,
                 init_seed=0, minibatch_size=64, checkpoint_every=0, checkpoint_path=""):
        self.obs_dim, self.num_actions, self.hidden_dim = obs_dim, num_actions, hidden_dim
        self.rollout_len, self.n_envs, self.gpu_minibatch_size = rollout_len, n_envs, gpu_minibatch_size
        self.gamma, self.gae_lambda, self.clip_epsilon = gamma, gae_lambda, clip_epsilon
        self.actor_lr, self.critic_lr, self.entropy_coef = actor_lr, critic_lr, entropy_coef
        self.value_loss_coef, self.num_epochs = value_loss_coef, num_epochs
        self.normalize_advantages, self.target_kl, self.max_grad_norm = normalize_advantages, target_kl, max_grad_norm
        self.anneal_lr, self.anneal_entropy, self.target_total_steps = anneal_lr, anneal_entropy, target_total_steps
        self.clip_value, self.norm_adv_per_minibatch, self.init_seed = clip_value, norm_adv_per_minibatch, init_seed
        # minibatch_size is the CPU trainer's; it is carried for the checkpoint metadata only
        self.minibatch_size, self.checkpoint_every, self.checkpoint_path = minibatch_size, checkpoint_every, checkpoint_path
        self.train_step_count = 0
        self.actor = self.critic = self.rb = self.upd = None

    def _nets(self):
        H = self.hidden_dim
        return (seq(LinearReLU(self.obs_dim, H), LinearReLU(H, H), Linear(H, self.num_actions)),
                seq(LinearReLU(self.obs_dim, H), LinearReLU(H, H), Linear(H, 1)))

    def build_networks(self, ctx):
        """Create and initialise actor and critic on `ctx` (a no-op once they exist)."""
        if self.actor is None:
            am, cm = self._nets()
            self.actor = Network(ctx, am, Adam(lr=self.actor_lr), Xavier(seed=2 * self.init_seed + 1))
            self.critic = Network(ctx, cm, Adam(lr=self.critic_lr), Xavier(seed=2 * self.init_seed + 2))

    def save_checkpoint(self, filepath):
        """ppo.mojo:3926-3980."""
        checkpoint.save_ppo_agent(self, filepath)

    def load_checkpoint(self, filepath, ctx=None):
        """ppo.mojo:3982-4055.  `ctx` is needed when the networks have not been built yet."""
        self._networks_for_load(ctx)
        checkpoint.load_ppo_agent(self, filepath)

    def _networks_for_load(self, ctx):
        if self.actor is None:
            if ctx is None:
                raise ValueError("load_checkpoint: pass the DeviceContext, the networks do not exist yet")
            self.build_networks(ctx)

    def _build(self, ctx, env):
        self.build_networks(ctx)
        self.rb = ppo.RolloutBuffers(ctx, env, self.actor.model, self.critic.model, self.n_envs, self.rollout_len,
                                     done_cap=max(1024, 2 * self.n_envs * self.rollout_len // 8),
                                     continuous=self.continuous)
        self.rb.actor_params, self.rb.critic_params = self.actor.params, self.critic.params
        cls = ppo.ContinuousUpdate if self.continuous else ppo.DiscreteUpdate
        self.upd = cls(ctx, self.rb, self.gpu_minibatch_size, self.actor.optimizer, self.critic.optimizer,
                       gamma=self.gamma, gae_lambda=self.gae_lambda, clip_epsilon=self.clip_epsilon,
                       entropy_coef=self.entropy_coef, value_loss_coef=self.value_loss_coef,
                       max_grad_norm=self.max_grad_norm, clip_value=self.clip_value,
                       normalize_advantages=self.normalize_advantages,
                       norm_adv_per_minibatch=self.norm_adv_per_minibatch, target_kl=self.target_kl,
                       normalize_rewards=getattr(self, "normalize_rewards", False))
        # the optimiser state lives with the update object; share the networks' buffers
        self.upd.actor_state, self.upd.critic_state = self.actor.optimizer_state, self.critic.optimizer_state
        self.upd.actor_grads, self.upd.critic_grads = self.actor.grads, self.critic.grads


class DeepPPOContinuousAgent(DeepPPOAgent):
    """deep_agents/ppo/ppo_continuous.mojo:171-390: tanh hidden layers, StochasticActor head
    (state-independent log_std, small initial weights), Kaiming initialisation, critic gradient
    (V - R) / MB, optional reward normalisation."""
    continuous = True

    def __init__(self, obs_dim, action_dim, hidden_dim=64, rollout_len=128, n_envs=1024,
                 gpu_minibatch_size=256, normalize_rewards=True, entropy_coef=0.01, num_epochs=10,
                 target_kl=0.02, action_scale=1.0, action_bias=0.0, obs_noise_std=0.0, **kw):
        # defaults of ppo_continuous.mojo:236-266 where they differ from the discrete agent's
        super().__init__(obs_dim, action_dim, hidden_dim, rollout_len, n_envs, gpu_minibatch_size,
                         entropy_coef=entropy_coef, num_epochs=num_epochs, target_kl=target_kl, **kw)
        self.action_dim, self.normalize_rewards = action_dim, normalize_rewards
        # action_scale / action_bias only enter the reference's host-side evaluation (:661, :1514);
        # they are carried for callers that do the same
        self.action_scale, self.action_bias = action_scale, action_bias
        self.obs_noise_std = obs_noise_std

    def _nets(self):
        H = self.hidden_dim
        return (seq(LinearTanh(self.obs_dim, H), LinearTanh(H, H), StochasticActor(H, self.action_dim)),
                seq(LinearTanh(self.obs_dim, H), LinearTanh(H, H), Linear(H, 1)))

    def build_networks(self, ctx):
        if self.actor is None:
            am, cm = self._nets()
            self.actor = Network(ctx, am, Adam(lr=self.actor_lr), Kaiming(seed=2 * self.init_seed + 1))
            self.critic = Network(ctx, cm, Adam(lr=self.critic_lr), Kaiming(seed=2 * self.init_seed + 2))
            H = self.hidden_dim
            init_params_small(ctx, self.actor.params, self.obs_dim * H + H + H * H + H, H, self.action_dim,
                              seed=2 * self.init_seed + 3)

    def save_checkpoint(self, filepath):
        """ppo_continuous.mojo:493-523."""
        checkpoint.save_ppo_continuous_agent(self, filepath)

    def load_checkpoint(self, filepath, ctx=None):
        """ppo_continuous.mojo:525-604."""
        self._networks_for_load(ctx)
        checkpoint.load_ppo_continuous_agent(self, filepath)
