"""Stateless layers behind the reference's `Model` trait (deep_rl/model/model.mojo:30-273).

A model exposes the compile-time constants IN_DIM / OUT_DIM / PARAM_SIZE / CACHE_SIZE /
WORKSPACE_SIZE_PER_SAMPLE and the three GPU entry points the PPO agents call:
    forward_gpu_no_cache_ws[BATCH](ctx, output, input, params, workspace)
    forward_gpu_ws[BATCH](ctx, output, input, params, cache, workspace)
    backward_gpu_ws[BATCH](ctx, grad_input, grad_output, params, cache, grads, workspace)
`seq(l0, l1, l2)` builds the reference's Seq2[Seq2[L0, L1], L2] nest
(deep_rl/model/sequential.mojo:867-953): params are [L0 | L1 | L2], the cache is blocked per
layer [BATCH x CACHE_i].  The workspace argument is accepted for signature compatibility and
never touched: intermediate activations live in a library-owned buffer.
"""
import ctypes as C

from . import _lib
from .context import _ptr


class Model:
    def __init__(self, layers):
        self.layers = list(layers)          # (kind, in_dim, out_dim) of the leaf layers
        self.desc = _lib.make_desc(self.layers)
        self.IN_DIM = self.layers[0][1]
        self.OUT_DIM = _lib.call("mrl_mlp_out_dim", C.byref(self.desc))
        self.PARAM_SIZE = _lib.call("mrl_mlp_param_size", C.byref(self.desc))
        self.CACHE_SIZE = _lib.call("mrl_mlp_cache_size", C.byref(self.desc))
        # what the reference's Seq2 nest would ask for (inter-layer buffers), kept so that callers
        # sizing their workspace from it keep working
        self.WORKSPACE_SIZE_PER_SAMPLE = sum(
            (2 * o if k == _lib.STOCHASTIC_ACTOR else o) for k, _, o in self.layers[:-1])

    def _batch(self, input_buf):
        n = input_buf.numel()
        if n % self.IN_DIM:
            raise _lib.MrlError("input of %d floats is not a multiple of IN_DIM=%d" % (n, self.IN_DIM))
        return n // self.IN_DIM

    def _check(self, batch, output=None, params=None, cache=None, grads=None):
        for name, t, want in (("output", output, batch * self.OUT_DIM), ("params", params, self.PARAM_SIZE),
                              ("cache", cache, batch * self.CACHE_SIZE), ("grads", grads, self.PARAM_SIZE)):
            if t is not None and t.numel() < want:
                raise _lib.MrlError("%s buffer holds %d floats, need %d" % (name, t.numel(), want))

    def forward_gpu_no_cache_ws(self, ctx, output_buf, input_buf, params_buf, workspace_buf=None):
        b = self._batch(input_buf)
        self._check(b, output_buf, params_buf)
        _lib.call("mrl_mlp_forward", ctx.handle, C.byref(self.desc), b, _ptr(input_buf),
                  _ptr(params_buf), _ptr(output_buf), None)

    def forward_gpu_ws(self, ctx, output_buf, input_buf, params_buf, cache_buf, workspace_buf=None):
        b = self._batch(input_buf)
        self._check(b, output_buf, params_buf, cache_buf)
        _lib.call("mrl_mlp_forward", ctx.handle, C.byref(self.desc), b, _ptr(input_buf),
                  _ptr(params_buf), _ptr(output_buf), _ptr(cache_buf))

    def backward_gpu_ws(self, ctx, grad_input_buf, grad_output_buf, params_buf, cache_buf, grads_buf,
                        workspace_buf=None):
        n = grad_output_buf.numel()
        if n % self.OUT_DIM:
            raise _lib.MrlError("grad_output of %d floats is not a multiple of OUT_DIM=%d" % (n, self.OUT_DIM))
        b = n // self.OUT_DIM
        self._check(b, None, params_buf, cache_buf, grads_buf)
        _lib.call("mrl_mlp_backward", ctx.handle, C.byref(self.desc), b, _ptr(grad_output_buf),
                  _ptr(params_buf), _ptr(cache_buf), _ptr(grads_buf), _ptr(grad_input_buf))


def Linear(in_dim, out_dim):            # deep_rl/model/linear.mojo
    return Model([(_lib.LINEAR, in_dim, out_dim)])


def LinearReLU(in_dim, out_dim):        # deep_rl/model/linear_relu.mojo
    return Model([(_lib.LINEAR_RELU, in_dim, out_dim)])


def LinearTanh(in_dim, out_dim):        # deep_rl/model/linear_tanh.mojo
    return Model([(_lib.LINEAR_TANH, in_dim, out_dim)])


def StochasticActor(in_dim, action_dim):  # deep_rl/model/stochastic_actor.mojo
    return Model([(_lib.STOCHASTIC_ACTOR, in_dim, action_dim)])


def seq(*models):
    """Chain models; the flat layer list is what Seq2[Seq2[a, b], c] reduces to."""
    layers = []
    for m in models:
        layers.extend(m.layers)
    return Model(layers)
