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
