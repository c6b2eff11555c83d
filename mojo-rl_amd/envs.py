"""Batched environments behind the reference's GPUDiscreteEnv / GPUContinuousEnv traits.

core/env_traits.mojo:230-397 declares, per environment type, the compile-time constants
STATE_SIZE / OBS_DIM / NUM_ACTIONS / ACTION_DIM and three static methods
    step_kernel_gpu[BATCH, STATE_SIZE, OBS_DIM](ctx, states, actions, rewards, dones, obs, rng_seed)
    reset_kernel_gpu[BATCH, STATE_SIZE](ctx, states, rng_seed)
    selective_reset_kernel_gpu[BATCH, STATE_SIZE](ctx, states, dones, rng_seed)
over flat fp32 device buffers.  The classes below keep those names and argument meanings; the
compile-time BATCH becomes the leading size of the buffers.  All calls only enqueue.
"""
import collections

import torch

from . import _lib
from .context import _ptr

# core/vec_env.mojo:25-58: the batched result of one step (observations per env, rewards, done flags).
# The reference fills it from SIMD vectors on the host; here the three members are the device tensors
# the step wrote ([batch, OBS_DIM], [batch], [batch]; done flags are 0.0 / 1.0 floats as in the traits).
VecStepResult = collections.namedtuple("VecStepResult", ["observations", "rewards", "dones"])


class _GPUEnv:
    ENV_ID = -1
    STATE_SIZE = 0
    OBS_DIM = 0
    NUM_ACTIONS = 0   # discrete envs
    ACTION_DIM = 0    # continuous envs

    @classmethod
    def _batch(cls, states):
        n = states.numel()
        if n % cls.STATE_SIZE:
            raise _lib.MrlError("states buffer of %d floats is not a multiple of STATE_SIZE=%d"
                                % (n, cls.STATE_SIZE))
        return n // cls.STATE_SIZE

    @classmethod
    def _check(cls, batch, actions=None, rewards=None, dones=None, obs=None):
        aw = cls.ACTION_DIM if cls.ACTION_DIM else 1
        for name, t, want in (("actions", actions, batch * aw), ("rewards", rewards, batch),
                              ("dones", dones, batch), ("obs", obs, batch * cls.OBS_DIM)):
            if t is not None and t.numel() != want:
                raise _lib.MrlError("%s buffer holds %d floats, expected %d" % (name, t.numel(), want))

    @classmethod
    def step_kernel_gpu(cls, ctx, states, actions, rewards, dones, obs, rng_seed=0):
        b = cls._batch(states)
        cls._check(b, actions, rewards, dones, obs)
        _lib.call("mrl_env_step", ctx.handle, cls.ENV_ID, b, _ptr(states), _ptr(actions),
                  _ptr(rewards), _ptr(dones), _ptr(obs), int(rng_seed) & (2**64 - 1))

    @classmethod
    def reset_kernel_gpu(cls, ctx, states, rng_seed=0):
        _lib.call("mrl_env_reset", ctx.handle, cls.ENV_ID, cls._batch(states), _ptr(states),
                  int(rng_seed) & (2**64 - 1))

    @classmethod
    def selective_reset_kernel_gpu(cls, ctx, states, dones, rng_seed):
        b = cls._batch(states)
        cls._check(b, dones=dones)
        _lib.call("mrl_env_selective_reset", ctx.handle, cls.ENV_ID, b, _ptr(states), _ptr(dones),
                  int(rng_seed) & (2**64 - 1))

    @classmethod
    def step_autoreset_kernel_gpu(cls, ctx, states, actions, rewards, dones, obs, step_seed=0,
                                  reset_seed=0):
        """step_kernel_gpu, selective_reset_kernel_gpu and the obs extraction in one launch."""
        b = cls._batch(states)
        cls._check(b, actions, rewards, dones, obs)
        _lib.call("mrl_env_step_autoreset", ctx.handle, cls.ENV_ID, b, _ptr(states), _ptr(actions),
                  _ptr(rewards), _ptr(dones), _ptr(obs), int(step_seed) & (2**64 - 1),
                  int(reset_seed) & (2**64 - 1))


    @classmethod
    def step_result(cls, ctx, states, actions, rng_seed=0):
        """step_kernel_gpu into fresh buffers, returned as a VecStepResult."""
        b = cls._batch(states)
        rewards, dones = ctx.enqueue_create_buffer(b), ctx.enqueue_create_buffer(b)
        obs = ctx.enqueue_create_buffer(b * cls.OBS_DIM)
        cls.step_kernel_gpu(ctx, states, actions, rewards, dones, obs, rng_seed)
        return VecStepResult(obs.view(b, cls.OBS_DIM), rewards, dones)


class CartPoleEnv(_GPUEnv):           # envs/cartpole.mojo:120
    ENV_ID, STATE_SIZE, OBS_DIM, NUM_ACTIONS = _lib.ENV_CARTPOLE, 4, 4, 2

    @classmethod
    def bind_step_counters(cls, ctx, states, steps):
        """Makes the int32 device tensor `steps` (one entry per env, or None to forget the binding) the
        per-env step counters behind the 500-step truncation for the rows at `states`; without it the
        context keeps counters of its own per states pointer."""
        from .context import _ptr
        if steps is not None and (steps.dtype != torch.int32 or steps.numel() * cls.STATE_SIZE != states.numel()):
            raise _lib.MrlError("step counters: one int32 per env")
        _lib.call("mrl_cartpole_bind_steps", ctx.handle, _ptr(states), states.numel() // cls.STATE_SIZE, _ptr(steps))


class PendulumV2(_GPUEnv):            # envs/pendulum/pendulum_v2.mojo:57
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_PENDULUM, 8, 3, 1


class LunarLanderV2(_GPUEnv):         # envs/lunar_lander/lunar_lander_v2.mojo:123
    ENV_ID, STATE_SIZE, OBS_DIM, NUM_ACTIONS = _lib.ENV_LUNARLANDER, 192, 8, 4

    @staticmethod
    def set_wind(ctx, enable, wind_power=15.0, turbulence_power=1.5):
        """The struct parameters ENABLE_WIND / WIND_POWER / TURBULENCE_POWER (lunar_lander_v2.mojo:123-127)
        as a setting of the context, shared by both action forms, for steps enqueued from now on."""
        _lib.call("mrl_lunar_set_wind", ctx.handle, int(bool(enable)), float(wind_power), float(turbulence_power))


class LunarLanderV2Continuous(_GPUEnv):
    """LunarLanderV2 as a GPUContinuousEnv (the reference overloads step_kernel_gpu on the one
    struct by ACTION_DIM, lunar_lander_v2.mojo:1520-1588; here the overload is a class of its
    own): action[0] main throttle in [-1, 1], action[1] side control in [-1, 1]."""
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_LUNARLANDER_CONTINUOUS, 192, 8, 2
    set_wind = LunarLanderV2.set_wind


class BipedalWalkerV2(_GPUEnv):       # envs/bipedal_walker/bipedal_walker_v2.mojo:103
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_BIPEDAL, 950, 24, 4


class HalfCheetahPlanarV2(_GPUEnv):   # envs/half_cheetah/cheetah_planar_v2.mojo:91
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_HALFCHEETAH, 253, 17, 6


class CarRacingV2(_GPUEnv):           # envs/car_racing/car_racing_v2.mojo:90
    """State-based CarRacing: 13-float observation (hull pose and velocity, front wheel angles, wheel
    spins, speed), action [steering, gas, brake] in [-1, 1]; every row carries its own random track."""
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_CARRACING, 3040, 13, 3
    STEP_CPU_ENV, STEP_GPU_TRAIT = 0, 1

    @staticmethod
    def set_step_form(ctx, form):
        """Which of the reference's two steps the context's CarRacingV2 steps follow from now on:
        STEP_CPU_ENV (default; CarRacingV2.step, car_racing_v2.mojo:258-287: reward -0.1 + 100 / tiles,
        Float64) or STEP_GPU_TRAIT (step_kernel_gpu, :1556-1716, what the reference's train_gpu runs:
        reward 0.5 * forward speed - 0.01 + 100 / tiles, fp32).  Dynamics and observations are the same."""
        _lib.call("mrl_car_racing_set_step_form", ctx.handle, int(form))


class HopperPlanar(_GPUEnv):          # envs/mujoco_planar/hopper_planar.mojo:162
    """The reference's planar Hopper (a Float64 CPU struct with a simplified physics of its own: 4 bodies,
    3 joints, observation 11, action 3) behind the batched env calls.  The reference has no GPU form of
    it; the row is this library's: the fp32 observation, one float of padding, then the struct's Float64
    state as pairs of floats (include/mrl.h at MRL_ENV_HOPPER_PLANAR)."""
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_HOPPER_PLANAR, 62, 11, 3


class Walker2dPlanar(_GPUEnv):        # envs/mujoco_planar/walker_planar.mojo:168
    """The reference's planar Walker2d (7 bodies, 6 joints, observation 17, action 6), as HopperPlanar."""
    ENV_ID, STATE_SIZE, OBS_DIM, ACTION_DIM = _lib.ENV_WALKER2D_PLANAR, 98, 17, 6
