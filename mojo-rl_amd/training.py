"""`Network` (deep_rl/training/network.mojo:92-126) and the weight initialisers
(deep_rl/initializer/initializers.mojo:51-104) on device buffers.

A Network owns the flat parameter, gradient and optimiser-state buffers of one model.  The
initialisers keep the reference's distributions -- a uniform fill of the WHOLE flat vector
(biases included) with bound sqrt(2 / (IN_DIM + OUT_DIM)) (Xavier) or sqrt(2 / IN_DIM)
(Kaiming), fan-in / fan-out being the network's input and output widths -- but draw from the
library's Philox stream: the reference draws from Mojo's process-global random_float64(), which
cannot be reproduced outside a Mojo runtime.
"""
import math

import torch

from . import _lib, checkpoint
from .context import _ptr


def _fill(ctx, buf, n, lo, hi, seed):
    _lib.call("mrl_init_uniform", ctx.handle, _ptr(buf), n, float(lo), float(hi), int(seed) & (2**64 - 1))


class Xavier:
    """U(+-sqrt(2 / (fan_in + fan_out))), initializers.mojo:69-76."""

    def __init__(self, seed=0):
        self.seed = seed

    def init(self, ctx, params, size, fan_in, fan_out):
        b = math.sqrt(2.0 / float(fan_in + fan_out))
        _fill(ctx, params, size, -b, b, self.seed)


class Kaiming:
    """U(+-sqrt(2 / fan_in)), initializers.mojo:97-104."""

    def __init__(self, seed=0):
        self.seed = seed

    def init(self, ctx, params, size, fan_in, fan_out):
        b = math.sqrt(2.0 / float(fan_in))
        _fill(ctx, params, size, -b, b, self.seed)


def init_params_small(ctx, params, offset, in_dim, action_dim, weight_scale=0.01, log_std_init=-0.5,
                      seed=0):
    """StochasticActor.init_params_small (deep_rl/model/stochastic_actor.mojo:95-128) applied to
    the head that starts `offset` floats into `params`: W_mean ~ U(+-weight_scale), b_mean = 0,
    log_std = log_std_init."""
    w = in_dim * action_dim
    head = params[offset:offset + w + 2 * action_dim]
    _fill(ctx, head, w, -weight_scale, weight_scale, seed)
    head[w:w + action_dim].zero_()
    head[w + action_dim:].fill_(log_std_init)


class Network:
    """model + optimiser + flat device buffers (params, grads, optimiser state)."""

    def __init__(self, ctx, model, optimizer, initializer):
        self.ctx, self.model, self.optimizer, self.initializer = ctx, model, optimizer, initializer
        dev = ctx.device
        self.params = torch.zeros(model.PARAM_SIZE, device=dev)
        self.grads = torch.zeros(model.PARAM_SIZE, device=dev)
        self.optimizer_state = torch.zeros(model.PARAM_SIZE * optimizer.STATE_PER_PARAM, device=dev)
        initializer.init(ctx, self.params, model.PARAM_SIZE, model.IN_DIM, model.OUT_DIM)

    def forward_gpu(self, output_buf, input_buf, cache_buf=None):
        if cache_buf is None:
            self.model.forward_gpu_no_cache_ws(self.ctx, output_buf, input_buf, self.params)
        else:
            self.model.forward_gpu_ws(self.ctx, output_buf, input_buf, self.params, cache_buf)

    def backward_gpu(self, grad_input_buf, grad_output_buf, cache_buf):
        self.model.backward_gpu_ws(self.ctx, grad_input_buf, grad_output_buf, self.params, cache_buf,
                                   self.grads)

    def update_gpu(self):
        self.optimizer.step_gpu(self.ctx, self.params, self.grads, self.optimizer_state)

    def save_checkpoint(self, filepath):
        """deep_rl/training/network.mojo:774-798."""
        checkpoint.save_network(self, filepath)

    def load_checkpoint(self, filepath):
        """deep_rl/training/network.mojo:800-835."""
        checkpoint.load_network(self, filepath)
