"""Adam behind the reference's `Optimizer` trait (deep_rl/optimizer/optimizer.mojo:51-68,
deep_rl/optimizer/adam.mojo).  `t` and `lr` live on the host object, as in the reference (the
PPO agent anneals `lr` between rollouts); state is [PARAM_SIZE, 2] interleaved (m, v)."""
from . import _lib
from .context import _ptr


class Adam:
    STATE_PER_PARAM = 2

    def __init__(self, lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8):
        self.lr, self.beta1, self.beta2, self.eps, self.t = lr, beta1, beta2, eps, 0

    def step_gpu(self, ctx, params_buf, grads_buf, state_buf):
        n = params_buf.numel()
        if grads_buf.numel() != n or state_buf.numel() != 2 * n:
            raise _lib.MrlError("Adam.step_gpu: grads must hold n and state 2n floats")
        self.t += 1
        _lib.call("mrl_adam_step", ctx.handle, _ptr(params_buf), _ptr(grads_buf), _ptr(state_buf), n,
                  self.t, self.lr, self.beta1, self.beta2, self.eps)
