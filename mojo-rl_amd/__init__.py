"""MI355X-native rollout / PPO-update path for mojo-rl, behind the reference's own interfaces.

The compute lives in libmrl_hip.so (hand-written gfx950 kernels, C ABI in include/mrl.h);
this package is the host-side mirror of the reference's env / model / optimizer traits.
Importing it loads the library and fails loudly if it is missing.
"""
from . import _lib
from ._lib import MrlError, LINEAR, LINEAR_RELU, LINEAR_TANH, STOCHASTIC_ACTOR

_lib.lib()  # load now: a missing or unloadable HIP library is an import error, not a fallback

from .context import DeviceContext  # noqa: E402
from .envs import (CartPoleEnv, PendulumV2, LunarLanderV2, LunarLanderV2Continuous, BipedalWalkerV2,  # noqa: E402
                   HalfCheetahPlanarV2, CarRacingV2, HopperPlanar, Walker2dPlanar, VecStepResult)
from .model import Model, Linear, LinearReLU, LinearTanh, StochasticActor, seq  # noqa: E402
from .optimizer import Adam  # noqa: E402
from .training import Network, Xavier, Kaiming, init_params_small  # noqa: E402
from . import ppo, checkpoint  # noqa: E402
from .agents import DeepPPOAgent, DeepPPOContinuousAgent, TrainingMetrics  # noqa: E402

__all__ = ["DeviceContext", "CartPoleEnv", "PendulumV2", "LunarLanderV2", "LunarLanderV2Continuous", "BipedalWalkerV2",
           "HalfCheetahPlanarV2", "CarRacingV2", "HopperPlanar", "Walker2dPlanar", "VecStepResult", "MrlError", "Model",
           "Linear", "LinearReLU", "LinearTanh", "StochasticActor", "seq", "Adam", "ppo",
           "Network", "Xavier", "Kaiming", "init_params_small", "checkpoint",
           "DeepPPOAgent", "DeepPPOContinuousAgent", "TrainingMetrics",
           "LINEAR", "LINEAR_RELU", "LINEAR_TANH", "STOCHASTIC_ACTOR"]
