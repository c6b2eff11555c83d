"""PPO pieces of deep_agents/ppo (kernels of ppo.mojo / kernels.mojo and the host math of
train_gpu) as enqueue-only calls on device buffers, plus the fused rollout step."""
import ctypes as C

import torch

from . import _lib
from .context import _ptr


def sample_actions(ctx, logits, actions, log_probs, seed):
    """_sample_actions_kernel, deep_agents/ppo/ppo.mojo:4064-4123."""
    n = actions.numel()
    _lib.call("mrl_sample_categorical", ctx.handle, _ptr(logits), n, logits.numel() // max(n, 1),
              int(seed) & 0xFFFFFFFF, _ptr(actions), _ptr(log_probs))


def sample_continuous_actions(ctx, actor_output, actions, log_probs, seed):
    """_sample_continuous_actions_kernel, deep_agents/ppo/kernels.mojo:12-98."""
    n = log_probs.numel()
    _lib.call("mrl_sample_gaussian", ctx.handle, _ptr(actor_output), n, actions.numel() // max(n, 1),
              int(seed) & 0xFFFFFFFF, _ptr(actions), _ptr(log_probs))


def compute_gae(ctx, rewards, values, dones, bootstrap, gamma, gae_lambda, advantages, returns):
    """GAE over time-major [T*N] buffers (index t*N + env); ppo.mojo:2317-2353."""
    n = bootstrap.numel()
    _lib.call("mrl_gae", ctx.handle, rewards.numel() // n, n, _ptr(rewards), _ptr(values), _ptr(dones),
              _ptr(bootstrap), float(gamma), float(gae_lambda), _ptr(advantages), _ptr(returns))


def normalize_advantages(ctx, advantages):
    """(A - mean) / (sqrt(var + 1e-8) + 1e-8) in place; ppo.mojo:2356-2371, kernels.mojo:507-599."""
    _lib.call("mrl_normalize_advantages", ctx.handle, _ptr(advantages), advantages.numel())


def gather_minibatch(ctx, indices, rollout, minibatch, obs_dim, act_dim=1):
    """ppo_gather_minibatch_kernel (ppo.mojo:135-191).  rollout / minibatch: tuples of
    (obs, actions, advantages, returns, log_probs, values) buffers; indices int32."""
    if indices.dtype != torch.int32:
        raise _lib.MrlError("minibatch indices must be int32")
    _lib.call("mrl_gather_minibatch", ctx.handle, _ptr(indices), indices.numel(), obs_dim, act_dim,
              *[_ptr(t) for t in rollout], *[_ptr(t) for t in minibatch])


def ppo_actor_grad_with_kl(ctx, grad_logits, kl, logits, old_log_probs, advantages, actions,
                           clip_epsilon, entropy_coef):
    """ppo_actor_grad_with_kl_kernel, ppo.mojo:285-378 (outputs first, like the kernel)."""
    mb = actions.numel()
    _lib.call("mrl_ppo_actor_grad_discrete", ctx.handle, _ptr(logits), _ptr(old_log_probs),
              _ptr(advantages), _ptr(actions), mb, logits.numel() // max(mb, 1), float(clip_epsilon),
              float(entropy_coef), _ptr(grad_logits), _ptr(kl))


def ppo_continuous_actor_grad(ctx, grad_output, kl, actor_output, old_log_probs, advantages, actions,
                              clip_epsilon, entropy_coef):
    """ppo_continuous_actor_grad_kernel, kernels.mojo:230-412."""
    mb = old_log_probs.numel()
    _lib.call("mrl_ppo_actor_grad_gaussian", ctx.handle, _ptr(actor_output), _ptr(old_log_probs),
              _ptr(advantages), _ptr(actions), mb, actions.numel() // max(mb, 1), float(clip_epsilon),
              float(entropy_coef), _ptr(grad_output), _ptr(kl))


def ppo_critic_grad(ctx, grad_values, values, returns, value_loss_coef=0.5, old_values=None,
                    clip_epsilon=0.0, continuous=False):
    """ppo_critic_grad(_clipped)_kernel: discrete agent ppo.mojo:538-633 (2*c_v*(V-R)/MB),
    continuous agent kernels.mojo:416-486 ((V-R)/MB); clipped when old_values is given."""
    _lib.call("mrl_ppo_critic_grad", ctx.handle, _ptr(values), _ptr(old_values), _ptr(returns),
              returns.numel(), 1 if continuous else 0, 0 if old_values is None else 1,
              float(value_loss_coef), float(clip_epsilon), _ptr(grad_values))


def clip_grad_norm(ctx, grads, max_grad_norm):
    """gradient_norm + reduce + apply, ppo.mojo:382-534 / kernels.mojo:603-805."""
    _lib.call("mrl_clip_grad_norm", ctx.handle, _ptr(grads), grads.numel(), float(max_grad_norm))


def clamp_log_std_params(ctx, params, log_std_offset, action_dim):
    """clamp_log_std_params_kernel, kernels.mojo:842-873."""
    _lib.call("mrl_clamp_log_std", ctx.handle, _ptr(params), log_std_offset, action_dim)


class RolloutBuffers:
    """Device buffers of train_gpu's collection phase for a discrete-action env
    (deep_agents/ppo/ppo.mojo:1616-1775): time-major rollout arrays, per-env episode
    accumulators and the device-side list of finished episodes."""

    def __init__(self, ctx, env, actor, critic, n_envs, rollout_len, done_cap=None):
        dev = ctx.device
        z = lambda *s: torch.zeros(*s, device=dev)
        self.ctx, self.env, self.actor, self.critic = ctx, env, actor, critic
        self.n_envs, self.rollout_len = n_envs, rollout_len
        self.states = z(n_envs * env.STATE_SIZE)
        self.obs = z(n_envs * env.OBS_DIM)
        T = rollout_len
        self.r_obs = z(T * n_envs * env.OBS_DIM)
        self.r_actions, self.r_log_probs, self.r_values = z(T * n_envs), z(T * n_envs), z(T * n_envs)
        self.r_rewards, self.r_dones = z(T * n_envs), z(T * n_envs)
        self.ep_return, self.ep_length = z(n_envs), z(n_envs)
        self.done_cap = done_cap or max(1024, 4 * n_envs)
        self.done_returns, self.done_lengths = z(self.done_cap), z(self.done_cap)
        self.done_count = torch.zeros(1, dtype=torch.int32, device=dev)
        self.actor_params = None
        self.critic_params = None

    def descriptor(self):
        r = _lib.Rollout()
        e = self.env
        r.env_id, r.n_envs, r.obs_dim, r.num_actions = e.ENV_ID, self.n_envs, e.OBS_DIM, e.NUM_ACTIONS
        r.states, r.obs = _ptr(self.states), _ptr(self.obs)
        r.actor_params, r.critic_params = _ptr(self.actor_params), _ptr(self.critic_params)
        r.actor, r.critic = self.actor.desc, self.critic.desc
        r.r_obs, r.r_actions, r.r_log_probs = _ptr(self.r_obs), _ptr(self.r_actions), _ptr(self.r_log_probs)
        r.r_values, r.r_rewards, r.r_dones = _ptr(self.r_values), _ptr(self.r_rewards), _ptr(self.r_dones)
        r.ep_return, r.ep_length = _ptr(self.ep_return), _ptr(self.ep_length)
        r.done_returns, r.done_lengths = _ptr(self.done_returns), _ptr(self.done_lengths)
        r.done_count, r.done_cap = _ptr(self.done_count), self.done_cap
        return r


def rollout_step(ctx, desc, t, sample_seed, step_seed=0, reset_seed=0):
    """One pass of train_gpu's inner loop body (ppo.mojo:2069-2285), enqueue only."""
    _lib.call("mrl_rollout_step", ctx.handle, C.byref(desc), t, int(sample_seed) & 0xFFFFFFFF,
              int(step_seed) & (2**64 - 1), int(reset_seed) & (2**64 - 1))


class DiscreteUpdate:
    """Phases 2 and 3 of DeepPPOAgent.train_gpu (deep_agents/ppo/ppo.mojo:2296-2727) on device
    buffers: bootstrap value, GAE, advantage normalisation, then epochs of shuffled minibatches,
    each running actor forward / loss gradient / backward / clip / Adam and the same for the
    critic.  Nothing is copied to the host inside an epoch; the mean KL of the last minibatch is
    read once per epoch for the early-stop test."""

    def __init__(self, ctx, rb, minibatch, actor_opt, critic_opt, gamma=0.99, gae_lambda=0.95,
                 clip_epsilon=0.2, entropy_coef=0.01, value_loss_coef=0.5, max_grad_norm=0.5,
                 clip_value=True, normalize_advantages=True, norm_adv_per_minibatch=True,
                 target_kl=0.015):
        self.ctx, self.rb, self.mb = ctx, rb, minibatch
        self.actor_opt, self.critic_opt = actor_opt, critic_opt
        self.gamma, self.gae_lambda = gamma, gae_lambda
        self.clip_epsilon, self.entropy_coef, self.value_loss_coef = clip_epsilon, entropy_coef, value_loss_coef
        self.max_grad_norm, self.clip_value = max_grad_norm, clip_value
        self.normalize_advantages, self.norm_adv_per_minibatch = normalize_advantages, norm_adv_per_minibatch
        self.target_kl = target_kl
        dev = ctx.device
        z = lambda n: torch.zeros(n, device=dev)
        total = rb.n_envs * rb.rollout_len
        obs_dim, na = rb.env.OBS_DIM, rb.env.NUM_ACTIONS
        self.total = total
        self.advantages, self.returns, self.bootstrap = z(total), z(total), z(rb.n_envs)
        self.mb_obs, self.mb_actions = z(minibatch * obs_dim), z(minibatch)
        self.mb_adv, self.mb_ret, self.mb_logp, self.mb_val = z(minibatch), z(minibatch), z(minibatch), z(minibatch)
        self.logits, self.values = z(minibatch * na), z(minibatch)
        self.g_logits, self.g_values, self.kl = z(minibatch * na), z(minibatch), z(minibatch)
        self.actor_cache = z(minibatch * rb.actor.CACHE_SIZE)
        self.critic_cache = z(minibatch * rb.critic.CACHE_SIZE)
        self.actor_grads, self.critic_grads = z(rb.actor.PARAM_SIZE), z(rb.critic.PARAM_SIZE)
        self.actor_state, self.critic_state = z(2 * rb.actor.PARAM_SIZE), z(2 * rb.critic.PARAM_SIZE)

    def compute_advantages(self):
        rb, ctx = self.rb, self.ctx
        rb.critic.forward_gpu_no_cache_ws(ctx, self.bootstrap, rb.obs, rb.critic_params)
        compute_gae(ctx, rb.r_rewards, rb.r_values, rb.r_dones, self.bootstrap, self.gamma,
                    self.gae_lambda, self.advantages, self.returns)
        if self.normalize_advantages:
            normalize_advantages(ctx, self.advantages)

    def minibatch_step(self, indices):
        rb, ctx = self.rb, self.ctx
        gather_minibatch(ctx, indices,
                         (rb.r_obs, rb.r_actions, self.advantages, self.returns, rb.r_log_probs, rb.r_values),
                         (self.mb_obs, self.mb_actions, self.mb_adv, self.mb_ret, self.mb_logp, self.mb_val),
                         rb.env.OBS_DIM, 1)
        if self.norm_adv_per_minibatch:
            normalize_advantages(ctx, self.mb_adv)
        rb.actor.forward_gpu_ws(ctx, self.logits, self.mb_obs, rb.actor_params, self.actor_cache)
        ppo_actor_grad_with_kl(ctx, self.g_logits, self.kl, self.logits, self.mb_logp, self.mb_adv,
                               self.mb_actions, self.clip_epsilon, self.entropy_coef)
        rb.actor.backward_gpu_ws(ctx, None, self.g_logits, rb.actor_params, self.actor_cache, self.actor_grads)
        if self.max_grad_norm > 0.0:
            clip_grad_norm(ctx, self.actor_grads, self.max_grad_norm)
        self.actor_opt.step_gpu(ctx, rb.actor_params, self.actor_grads, self.actor_state)
        rb.critic.forward_gpu_ws(ctx, self.values, self.mb_obs, rb.critic_params, self.critic_cache)
        ppo_critic_grad(ctx, self.g_values, self.values, self.mb_ret, self.value_loss_coef,
                        self.mb_val if self.clip_value else None, self.clip_epsilon)
        rb.critic.backward_gpu_ws(ctx, None, self.g_values, rb.critic_params, self.critic_cache, self.critic_grads)
        if self.max_grad_norm > 0.0:
            clip_grad_norm(ctx, self.critic_grads, self.max_grad_norm)
        self.critic_opt.step_gpu(ctx, rb.critic_params, self.critic_grads, self.critic_state)

    def run_epoch(self, permutation):
        """permutation: int32 device tensor over the T*N samples; only whole minibatches are used
        (ppo.mojo:2438).  Returns the mean KL of the epoch's last minibatch."""
        n_mb = self.total // self.mb
        for k in range(n_mb):
            self.minibatch_step(permutation[k * self.mb:(k + 1) * self.mb])
        return float(self.kl.mean().item()) if self.target_kl > 0.0 else 0.0
