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


def add_obs_noise(ctx, obs, n_envs, noise_std, seed):
    """add_obs_noise_kernel, deep_agents/ppo/kernels.mojo:882-925: Gaussian noise of standard deviation
    noise_std on every entry of obs [n_envs, OBS_DIM], in place."""
    _lib.call("mrl_add_obs_noise", ctx.handle, _ptr(obs), n_envs, obs.numel() // max(n_envs, 1), float(noise_std),
              int(seed) & 0xFFFFFFFF)


def greedy_actions(ctx, actor_output, actions, n, continuous):
    """The actions of `n` rows without sampling: the Gaussian head's mean
    (extract_deterministic_actions, deep_agents/ppo/ppo_continuous.mojo:807-822; rows of
    actor_output are [mean | log_std]) or the argmax of the logits (select_action with
    training=False, ppo.mojo:988-1027)."""
    width = actor_output.numel() // max(n, 1)
    _lib.call("mrl_greedy_actions", ctx.handle, _ptr(actor_output), n, width // 2 if continuous else width,
              1 if continuous else 0, _ptr(actions))


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


CLIP_STATIC_MAX_N = 1 << 24


def clip_grad_norm_static(ctx, grads, max_grad_norm):
    """clip_grad_norm for callers that must not allocate device memory: the partial sums live in a
    file-scope device array of the library.  Same results; at most CLIP_STATIC_MAX_N elements; calls
    that overlap on one device race on that array."""
    _lib.call("mrl_clip_grad_norm_static", ctx.handle, _ptr(grads), grads.numel(), float(max_grad_norm))


def clamp_log_std_params(ctx, params, log_std_offset, action_dim):
    """clamp_log_std_params_kernel, kernels.mojo:842-873."""
    _lib.call("mrl_clamp_log_std", ctx.handle, _ptr(params), log_std_offset, action_dim)


def permutation(ctx, indices, seed):
    """Fills the int32 device buffer with a seeded pseudo-random permutation of 0..n-1; stands
    where train_gpu shuffles on the host (ppo.mojo:2425-2434)."""
    if indices.dtype != torch.int32:
        raise _lib.MrlError("permutation indices must be int32")
    _lib.call("mrl_permutation", ctx.handle, _ptr(indices), indices.numel(), int(seed) & (2**64 - 1))


def shuffle_indices(ctx, indices, uniforms, workspace=None):
    """shuffle_indices of core/utils/shuffle.mojo:21-48 on supplied draws: fills the int32 device buffer
    with the permutation that the reference's Fisher-Yates loop produces when iteration i = n-1 .. 1
    draws uniforms[n - 1 - i] (float64 device tensor of n - 1 values).  workspace: int32 device
    scratch of 2n + 1 entries, allocated here when not given."""
    n = indices.numel()
    if indices.dtype != torch.int32:
        raise _lib.MrlError("permutation indices must be int32")
    if n > 1 and (uniforms.dtype != torch.float64 or uniforms.numel() < n - 1):
        raise _lib.MrlError("shuffle_indices needs n - 1 float64 uniforms")
    if workspace is None:
        workspace = torch.empty(2 * n + 1, dtype=torch.int32, device=indices.device)
    elif workspace.dtype != torch.int32 or workspace.numel() < 2 * n + 1:
        raise _lib.MrlError("shuffle_indices needs an int32 workspace of 2n + 1 entries")
    _lib.call("mrl_permutation_from_uniforms", ctx.handle, _ptr(indices), n, _ptr(uniforms) if n > 1 else None,
              _ptr(workspace))
    return workspace


def minibatch_adv_stats(ctx, indices, advantages, minibatch, stats):
    """stats[2k], stats[2k + 1] = mean and sqrt(variance + 1e-8) of the advantages of minibatch k of
    `indices` (ppo.mojo:2478-2511): what the fused update normalises with."""
    n_mb = indices.numel() // minibatch
    if indices.dtype != torch.int32 or stats.numel() < 2 * n_mb:
        raise _lib.MrlError("minibatch_adv_stats needs int32 indices and 2 floats per minibatch")
    _lib.call("mrl_minibatch_adv_stats", ctx.handle, _ptr(indices), _ptr(advantages), minibatch, n_mb, _ptr(stats))


def kl_check(ctx, kl, target_kl, flag):
    """Device-side early-stop test: flag[0] (int32) becomes 1 when mean(kl) > target_kl and stays
    1; flag[1] holds the bits of the mean (ppo.mojo:2557-2573 without the host copy)."""
    _lib.call("mrl_kl_check", ctx.handle, _ptr(kl), kl.numel(), float(target_kl), _ptr(flag))


class RunningMeanStd:
    """core/utils/normalization.mojo:188-292 with the state (count, mean, var_sum) in device
    memory, Float64 throughout; used for reward normalisation (ppo_continuous.mojo:2867-2871)."""

    def __init__(self, ctx):
        self.ctx = ctx
        self.state = torch.zeros(3, dtype=torch.float64, device=ctx.device)

    def update(self, x):
        _lib.call("mrl_rms_update", self.ctx.handle, _ptr(self.state), _ptr(x), x.numel())

    def normalize(self, x):
        _lib.call("mrl_rms_normalize", self.ctx.handle, _ptr(self.state), _ptr(x), x.numel())


class RolloutBuffers:
    """Device buffers of train_gpu's collection phase (deep_agents/ppo/ppo.mojo:1616-1775,
    ppo_continuous.mojo:2180-2470): time-major rollout arrays, per-env episode accumulators and
    the device-side list of finished episodes.  A discrete agent (env.NUM_ACTIONS > 0 and
    continuous=False) stores one float per action, a continuous one env.ACTION_DIM."""

    def __init__(self, ctx, env, actor, critic, n_envs, rollout_len, done_cap=None, continuous=None):
        dev = ctx.device
        z = lambda *s: torch.zeros(*s, device=dev)
        self.ctx, self.env, self.actor, self.critic = ctx, env, actor, critic
        self.n_envs, self.rollout_len = n_envs, rollout_len
        self.continuous = (env.NUM_ACTIONS == 0) if continuous is None else continuous
        self.act_width = env.ACTION_DIM if self.continuous else 1
        self.states = z(n_envs * env.STATE_SIZE)
        self.obs = z(n_envs * env.OBS_DIM)
        T = rollout_len
        self.r_obs = z(T * n_envs * env.OBS_DIM)
        self.r_actions = z(T * n_envs * self.act_width)
        self.r_log_probs, self.r_values = z(T * n_envs), z(T * n_envs)
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
        r.env_id, r.n_envs, r.obs_dim = e.ENV_ID, self.n_envs, e.OBS_DIM
        r.num_actions = 0 if self.continuous else e.NUM_ACTIONS
        r.states, r.obs = _ptr(self.states), _ptr(self.obs)
        r.actor_params, r.critic_params = _ptr(self.actor_params), _ptr(self.critic_params)
        r.actor, r.critic = self.actor.desc, self.critic.desc
        r.r_obs, r.r_actions, r.r_log_probs = _ptr(self.r_obs), _ptr(self.r_actions), _ptr(self.r_log_probs)
        r.r_values, r.r_rewards, r.r_dones = _ptr(self.r_values), _ptr(self.r_rewards), _ptr(self.r_dones)
        r.ep_return, r.ep_length = _ptr(self.ep_return), _ptr(self.ep_length)
        r.done_returns, r.done_lengths = _ptr(self.done_returns), _ptr(self.done_lengths)
        r.done_count, r.done_cap = _ptr(self.done_count), self.done_cap
        return r


def policy_step(ctx, rb, t, sample_seed, actions):
    """Policy half of collection step t on rb.obs (actor + critic forward, sampling, pre-step store into
    rollout row t); `actions` [N * act_width] receives what the envs are to be stepped with.  Enqueue only."""
    N, od, aw = rb.n_envs, rb.env.OBS_DIM, rb.act_width
    name = "mrl_policy_step_gaussian" if rb.continuous else "mrl_policy_step_discrete"
    _lib.call(name, ctx.handle, C.byref(rb.actor.desc), C.byref(rb.critic.desc), N, _ptr(rb.obs),
              _ptr(rb.actor_params), _ptr(rb.critic_params), int(sample_seed) & 0xFFFFFFFF, _ptr(actions),
              _ptr(rb.r_obs[t * N * od:]), _ptr(rb.r_actions[t * N * aw:]), _ptr(rb.r_log_probs[t * N:]),
              _ptr(rb.r_values[t * N:]))


def rollout_step(ctx, desc, t, sample_seed, step_seed=0, reset_seed=0):
    """One pass of train_gpu's inner loop body (ppo.mojo:2069-2285, ppo_continuous.mojo:2619-2850),
    enqueue only."""
    _lib.call("mrl_rollout_step", ctx.handle, C.byref(desc), t, int(sample_seed) & 0xFFFFFFFF,
              int(step_seed) & (2**64 - 1), int(reset_seed) & (2**64 - 1))


def rollout_steps(ctx, desc, t0, n_steps, sample_seed, sample_stride, step_seed=0, step_stride=0,
                  reset_seed=0, reset_stride=0):
    """train_gpu's collection loop over steps t0 .. t0 + n_steps - 1, enqueue only: step t0 + k uses
    the seeds  seed + k * stride  (sample: mod 2^32, step / reset: mod 2^64).  One launch where the
    env and the networks allow it (the env rows then stay on chip for the whole range)."""
    _lib.call("mrl_rollout_steps", ctx.handle, C.byref(desc), t0, n_steps, int(sample_seed) & 0xFFFFFFFF,
              int(sample_stride) & 0xFFFFFFFF, int(step_seed) & (2**64 - 1), int(step_stride) & (2**64 - 1),
              int(reset_seed) & (2**64 - 1), int(reset_stride) & (2**64 - 1))


def rollout_fused(desc):
    """True when rollout_steps runs this descriptor as one launch per call."""
    return bool(_lib.call("mrl_rollout_fused", C.byref(desc)))


class PPOUpdate:
    """Phases 2 and 3 of train_gpu (deep_agents/ppo/ppo.mojo:2296-2727 for the discrete agent,
    ppo_continuous.mojo:2852-3260 for the continuous one) on device buffers: bootstrap value,
    optional reward normalisation, GAE, advantage normalisation, then epochs of shuffled
    minibatches, each one library call (mrl_ppo_update_minibatch / _epoch) that runs actor and
    critic forward / loss gradient / backward / clip / Adam (/ log_std clamp).  Nothing is copied
    to the host inside an epoch: the KL early-stop test runs on the device after every actor
    loss gradient, an update is not applied once it has fired (the reference's `break`), and
    the flag is read once per epoch."""

    def __init__(self, ctx, rb, minibatch, actor_opt, critic_opt, gamma=0.99, gae_lambda=0.95,
                 clip_epsilon=0.2, entropy_coef=0.01, value_loss_coef=0.5, max_grad_norm=0.5,
                 clip_value=True, normalize_advantages=True, norm_adv_per_minibatch=True,
                 target_kl=0.015, normalize_rewards=False):
        self.ctx, self.rb, self.mb = ctx, rb, minibatch
        self.actor_opt, self.critic_opt = actor_opt, critic_opt
        self.gamma, self.gae_lambda = gamma, gae_lambda
        self.clip_epsilon, self.entropy_coef, self.value_loss_coef = clip_epsilon, entropy_coef, value_loss_coef
        self.max_grad_norm, self.clip_value = max_grad_norm, clip_value
        self.normalize_advantages, self.norm_adv_per_minibatch = normalize_advantages, norm_adv_per_minibatch
        self.target_kl = target_kl
        self.continuous = rb.continuous
        self.reward_rms = RunningMeanStd(ctx) if normalize_rewards else None
        dev = ctx.device
        z = lambda n: torch.zeros(n, device=dev)
        total = rb.n_envs * rb.rollout_len
        obs_dim, aw = rb.env.OBS_DIM, rb.act_width
        head = rb.actor.OUT_DIM
        self.total = total
        self.advantages, self.returns, self.bootstrap = z(total), z(total), z(rb.n_envs)
        self.mb_obs, self.mb_actions = z(minibatch * obs_dim), z(minibatch * aw)
        self.mb_adv, self.mb_ret, self.mb_logp, self.mb_val = z(minibatch), z(minibatch), z(minibatch), z(minibatch)
        self.actor_out, self.values = z(minibatch * head), z(minibatch)
        self.g_actor_out, self.g_values, self.kl = z(minibatch * head), z(minibatch), z(minibatch)
        self.kl_flag = torch.zeros(4, dtype=torch.int32, device=dev)
        self.actor_cache = z(minibatch * rb.actor.CACHE_SIZE)
        self.critic_cache = z(minibatch * rb.critic.CACHE_SIZE)
        self.actor_grads, self.critic_grads = z(rb.actor.PARAM_SIZE), z(rb.critic.PARAM_SIZE)
        self.actor_state, self.critic_state = z(2 * rb.actor.PARAM_SIZE), z(2 * rb.critic.PARAM_SIZE)
        self.indices = torch.zeros(total, dtype=torch.int32, device=dev)
        self._t_base = (actor_opt.t, critic_opt.t)

    # names used by callers written against the discrete agent
    @property
    def logits(self):
        return self.actor_out

    @property
    def g_logits(self):
        return self.g_actor_out

    def descriptor(self):
        """The mrl_update view of this object (buffers, hyper-parameters, current learning rates)."""
        rb, u = self.rb, _lib.Update()
        u.minibatch, u.obs_dim, u.act_width = self.mb, rb.env.OBS_DIM, rb.act_width
        u.continuous = 1 if self.continuous else 0
        u.actor, u.critic = rb.actor.desc, rb.critic.desc
        for name, t in (("actor_params", rb.actor_params), ("critic_params", rb.critic_params),
                        ("actor_grads", self.actor_grads), ("critic_grads", self.critic_grads),
                        ("actor_state", self.actor_state), ("critic_state", self.critic_state),
                        ("r_obs", rb.r_obs), ("r_actions", rb.r_actions), ("r_log_probs", rb.r_log_probs),
                        ("r_values", rb.r_values), ("advantages", self.advantages), ("returns", self.returns),
                        ("mb_obs", self.mb_obs), ("mb_actions", self.mb_actions), ("mb_adv", self.mb_adv),
                        ("mb_ret", self.mb_ret), ("mb_logp", self.mb_logp), ("mb_val", self.mb_val),
                        ("actor_out", self.actor_out), ("values", self.values),
                        ("g_actor_out", self.g_actor_out), ("g_values", self.g_values), ("kl", self.kl),
                        ("actor_cache", self.actor_cache), ("critic_cache", self.critic_cache),
                        ("kl_flag", self.kl_flag)):
            setattr(u, name, _ptr(t))
        u.clip_epsilon, u.entropy_coef, u.value_loss_coef = self.clip_epsilon, self.entropy_coef, self.value_loss_coef
        u.max_grad_norm, u.target_kl = self.max_grad_norm, self.target_kl
        u.clip_value, u.norm_adv_per_minibatch = int(self.clip_value), int(self.norm_adv_per_minibatch)
        a, c = self.actor_opt, self.critic_opt
        if (a.beta1, a.beta2, a.eps) != (c.beta1, c.beta2, c.eps):
            raise _lib.MrlError("actor and critic optimisers must share beta1, beta2 and eps")
        u.actor_lr, u.critic_lr, u.beta1, u.beta2, u.eps = a.lr, c.lr, a.beta1, a.beta2, a.eps
        return u

    def compute_advantages(self):
        rb, ctx = self.rb, self.ctx
        rb.critic.forward_gpu_no_cache_ws(ctx, self.bootstrap, rb.obs, rb.critic_params)
        if self.reward_rms is not None:
            self.reward_rms.update(rb.r_rewards)
            self.reward_rms.normalize(rb.r_rewards)
        compute_gae(ctx, rb.r_rewards, rb.r_values, rb.r_dones, self.bootstrap, self.gamma,
                    self.gae_lambda, self.advantages, self.returns)
        if self.normalize_advantages:
            normalize_advantages(ctx, self.advantages)

    def reset_kl(self):
        """Clears the device flag and the applied-update counter (start of an update phase)."""
        self.kl_flag.zero_()
        self._t_base = (self.actor_opt.t, self.critic_opt.t)

    def minibatch_step(self, indices):
        if indices.dtype != torch.int32 or indices.numel() != self.mb:
            raise _lib.MrlError("minibatch_step needs %d int32 indices" % self.mb)
        u = self.descriptor()
        _lib.call("mrl_ppo_update_minibatch", self.ctx.handle, C.byref(u), _ptr(indices),
                  self.actor_opt.t + 1, self.critic_opt.t + 1)
        self.actor_opt.t += 1
        self.critic_opt.t += 1

    def kl_stopped(self):
        """Reads the device flag (one synchronising copy of 16 bytes): (stopped, last mean KL).
        When the stop has fired the optimisers' step counters are set to the updates applied."""
        f = self.kl_flag.cpu()
        stopped = bool(f[0].item())
        if stopped:
            applied = int(f[2].item())
            self.actor_opt.t = self._t_base[0] + applied
            self.critic_opt.t = self._t_base[1] + applied
        return stopped, float(f[1:2].view(torch.float32).item())

    def run_epoch(self, permutation_or_seed):
        """permutation_or_seed: an int32 device tensor over the T*N samples, or an int seed from
        which the permutation is drawn on the device.  Only whole minibatches are used
        (ppo.mojo:2438).  Returns (stopped, mean KL of the last minibatch tested)."""
        if isinstance(permutation_or_seed, int):
            permutation(self.ctx, self.indices, permutation_or_seed)
            perm = self.indices
        else:
            perm = permutation_or_seed
            if perm.dtype != torch.int32:
                raise _lib.MrlError("permutation must be int32")
        n_mb = min(self.total, perm.numel()) // self.mb
        u = self.descriptor()
        _lib.call("mrl_ppo_update_epoch", self.ctx.handle, C.byref(u), _ptr(perm), n_mb,
                  self.actor_opt.t, self.critic_opt.t)
        self.actor_opt.t += n_mb
        self.critic_opt.t += n_mb
        return self.kl_stopped() if self.target_kl > 0.0 else (False, 0.0)

    def update(self, num_epochs, seed=0):
        """compute_advantages + up to num_epochs epochs; stops after the epoch in which the KL
        flag was raised.  Returns the number of epochs run."""
        self.reset_kl()
        self.compute_advantages()
        for epoch in range(num_epochs):
            stopped, _ = self.run_epoch(int(seed) * 1000003 + epoch)
            if stopped:
                return epoch + 1
        return num_epochs


class DiscreteUpdate(PPOUpdate):
    """PPOUpdate for DeepPPOAgent (discrete actions, critic gradient 2*c_v*(V-R)/MB)."""


class ContinuousUpdate(PPOUpdate):
    """PPOUpdate for DeepPPOContinuousAgent (Gaussian actor with a StochasticActor head, critic
    gradient (V-R)/MB, log_std clamp after every actor step, optional reward normalisation)."""
