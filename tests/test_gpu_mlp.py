"""GPU parity: MLP forward / backward through the C ABI against the CPU oracle (serial fp32 loops
of the reference layers) and a torch fp32 reference.  Bar: outputs and gradients within 1e-4
relative (floor 1e-5 absolute, scaled by the magnitude of the tensor)."""
import sys

import zlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
RELU, TANH, LIN, ACTOR = 1, 2, 0, 3


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def mk(mrl, spec):
    f = {RELU: mrl.LinearReLU, TANH: mrl.LinearTanh, LIN: mrl.Linear, ACTOR: mrl.StochasticActor}
    return mrl.seq(*[f[k](i, o) for k, i, o in spec])


def close(got, want, what):
    scale = max(1.0, float(np.abs(want).max()))
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5 * scale, err_msg=what)


CASES = [
    ("lunar actor", [(RELU, 8, 256), (RELU, 256, 256), (LIN, 256, 4)], 300),
    ("lunar critic", [(RELU, 8, 256), (RELU, 256, 256), (LIN, 256, 1)], 257),
    ("cartpole actor", [(RELU, 4, 64), (RELU, 64, 64), (LIN, 64, 2)], 129),
    ("pendulum actor", [(TANH, 3, 64), (TANH, 64, 64), (ACTOR, 64, 1)], 200),
    ("cheetah actor", [(TANH, 17, 256), (TANH, 256, 256), (ACTOR, 256, 6)], 96),
    ("bipedal critic", [(TANH, 24, 256), (TANH, 256, 256), (LIN, 256, 1)], 64),
    ("odd sizes", [(RELU, 5, 33), (TANH, 33, 70), (LIN, 70, 3)], 37),
    ("single layer", [(LIN, 7, 5)], 1),
]


@pytest.mark.parametrize("name,spec,batch", CASES, ids=[c[0] for c in CASES])
def test_forward_backward_parity(mrl, orc, orcmod, ctx, name, spec, batch):
    say("mlp case", name, batch)
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    model = mk(mrl, spec)
    ls = orcmod.layers(spec)
    P, CS, OD = model.PARAM_SIZE, model.CACHE_SIZE, model.OUT_DIM
    assert P == orc.orc_mlp_param_size(ls, len(spec)) and CS == orc.orc_mlp_cache_size(ls, len(spec))
    fan = np.sqrt(2.0 / spec[0][1])
    params = rng.uniform(-fan, fan, P).astype(np.float32) * 0.7
    x = rng.normal(size=(batch, spec[0][1])).astype(np.float32)
    go = rng.normal(size=(batch, OD)).astype(np.float32)

    out_h = np.zeros((batch, OD), np.float32); cache_h = np.zeros(batch * CS, np.float32)
    orc.orc_mlp_forward(ls, len(spec), batch, x, params, out_h, cache_h.ctypes.data)

    d = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    p_d, x_d, go_d = d(params), d(x.reshape(-1)), d(go.reshape(-1))
    out_d = torch.full((batch * OD,), 9.0, device="cuda"); out_nc = torch.full((batch * OD,), 9.0, device="cuda")
    cache_d = torch.full((batch * CS,), 9.0, device="cuda")
    grads_d = torch.full((P,), 9.0, device="cuda"); gin_d = torch.full((x.size,), 9.0, device="cuda")
    model.forward_gpu_no_cache_ws(ctx, out_nc, x_d, p_d)
    model.forward_gpu_ws(ctx, out_d, x_d, p_d, cache_d)
    model.backward_gpu_ws(ctx, gin_d, go_d, p_d, cache_d, grads_d)     # overwrites the 9.0s
    ctx.synchronize()
    close(out_d.cpu().numpy().reshape(batch, OD), out_h, "forward")
    assert torch.equal(out_d, out_nc)
    close(cache_d.cpu().numpy(), cache_h, "cache")
    # The oracle's backward runs on the cache the kernels wrote (just shown to agree with the
    # oracle's own): a ReLU pre-activation within an ulp of zero may round to either side in the
    # two forwards, and the gate it selects is a step function -- not a tolerance question.
    grads_h = np.zeros(P, np.float32); gin_h = np.zeros_like(x)
    orc.orc_mlp_backward(ls, len(spec), batch, go, params, cache_d.cpu().numpy(), grads_h, gin_h.ctypes.data)
    close(grads_d.cpu().numpy(), grads_h, "param grads")
    close(gin_d.cpu().numpy().reshape(x.shape), gin_h, "input grads")
    # backward without grad_input (what the PPO update asks for): three-layer nets of the agents'
    # shapes take the fused kernels here, which sum in another order than the per-layer ones
    grads2 = torch.full((P,), 9.0, device="cuda")
    model.backward_gpu_ws(ctx, None, go_d, p_d, cache_d, grads2)
    ctx.synchronize()
    close(grads2.cpu().numpy(), grads_h, "param grads (no input gradient)")


def test_forward_matches_torch_fp32_at_update_size(mrl, ctx):
    # minibatch of 4096 rows through the 256-wide nets against torch fp32 matmuls
    torch.manual_seed(0)
    model = mk(mrl, [(RELU, 8, 256), (RELU, 256, 256), (LIN, 256, 4)])
    B = 4096
    p = (torch.rand(model.PARAM_SIZE, device="cuda") - 0.5) * 0.2
    x = torch.randn(B, 8, device="cuda")
    W0, b0 = p[:2048].view(8, 256), p[2048:2304]
    W1, b1 = p[2304:2304 + 65536].view(256, 256), p[67840:68096]
    W2, b2 = p[68096:68096 + 1024].view(256, 4), p[69120:69124]
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    h1 = torch.relu(x @ W0 + b0); h2 = torch.relu(h1 @ W1 + b1); want = h2 @ W2 + b2
    out = torch.zeros(B * 4, device="cuda"); cache = torch.zeros(B * model.CACHE_SIZE, device="cuda")
    model.forward_gpu_ws(ctx, out, x.reshape(-1), p, cache)
    go = torch.randn(B, 4, device="cuda")
    grads = torch.zeros(model.PARAM_SIZE, device="cuda")
    model.backward_gpu_ws(ctx, None, go.reshape(-1), p, cache, grads)
    ctx.synchronize()
    torch.testing.assert_close(out.view(B, 4), want, rtol=1e-4, atol=1e-5)
    m2 = go @ W2.T * (h2 > 0); m1 = m2 @ W1.T * (h1 > 0)
    want_g = torch.cat([(x.T @ m1).reshape(-1), m1.sum(0), (h1.T @ m2).reshape(-1), m2.sum(0),
                        (h2.T @ go).reshape(-1), go.sum(0)])
    torch.backends.cuda.matmul.allow_tf32 = prev
    torch.testing.assert_close(grads, want_g, rtol=1e-4, atol=1e-4 * float(want_g.abs().max()))


@pytest.mark.parametrize("H", [32, 256])      # 32: the layer-by-layer kernels; 256: the fused tile kernels
def test_tanh_layer_keeps_relative_accuracy_for_small_arguments(mrl, ctx, H):
    """The hidden layers' tanh against (float)tanh((double)x) over a log-spaced sweep of both signs,
    1e-9 .. 12: absolute error below 3e-7 AND relative error below 2e-6 (the exp-based form alone
    cancels for small |x|: relative error 1e-3 at 1e-4, and 0 instead of x below 3e-8).  Read from the
    cache of the first LinearTanh layer of an 8 -> H -> H -> 1 net whose first layer passes column 0
    of the input through unchanged (weights 1, bias 0), for the layer-by-layer and the fused forward."""
    model = mk(mrl, [(TANH, 8, H), (TANH, H, H), (LIN, H, 1)])
    mags = np.concatenate([np.logspace(-9, np.log10(12.0), 2040), [0.125, np.nextafter(np.float32(0.125), 0), 0.0, 1.0]])
    x = np.concatenate([mags, -mags]).astype(np.float32)
    B = x.size
    assert B == 4088
    inp = np.zeros((B, 8), np.float32); inp[:, 0] = x
    p = np.zeros(model.PARAM_SIZE, np.float32)
    p[:H] = 1.0                                             # W0[0, :] = 1, every other weight and bias 0
    out = torch.zeros(B, device="cuda"); cache = torch.zeros(B * model.CACHE_SIZE, device="cuda")
    model.forward_gpu_ws(ctx, out, torch.from_numpy(inp.reshape(-1)).cuda(), torch.from_numpy(p).cuda(), cache)
    ctx.synchronize()
    y = cache[:B * (8 + H)].cpu().numpy().reshape(B, 8 + H)[:, 8:]       # layer 0: [input | tanh output] per row
    want = np.tanh(x.astype(np.float64)).astype(np.float32)
    for j in (0, H - 1):
        err = np.abs(y[:, j].astype(np.float64) - want)
        assert err.max() < 3e-7
        nz = want != 0
        assert (err[nz] / np.abs(want[nz])).max() < 2e-6, float((err[nz] / np.abs(want[nz])).max())
        assert np.array_equal(y[~nz, j], want[~nz])
        tiny = np.abs(x) < 1e-4
        np.testing.assert_array_equal(y[tiny, j], x[tiny])                # tanh x = x to fp32 there


def test_mlp_argument_errors(mrl, ctx):
    model = mk(mrl, [(RELU, 8, 16), (LIN, 16, 2)])
    p = torch.zeros(model.PARAM_SIZE, device="cuda")
    with pytest.raises(mrl.MrlError):
        model.forward_gpu_no_cache_ws(ctx, torch.zeros(4, device="cuda"), torch.zeros(9, device="cuda"), p)
    with pytest.raises(mrl.MrlError):
        model.forward_gpu_no_cache_ws(ctx, torch.zeros(1, device="cuda"), torch.zeros(8, device="cuda"), p)
    with pytest.raises(mrl.MrlError):
        mrl.seq(mrl.LinearReLU(8, 16), mrl.Linear(15, 2))       # dims do not chain
    model.forward_gpu_no_cache_ws(ctx, torch.zeros(0, device="cuda"), torch.zeros(0, device="cuda"), p)


def test_reserved_workspace_is_not_grown_again(mrl):
    """A context whose workspace was reserved ahead runs the layer-by-layer path without allocating:
    the size it reports stays what was reserved, and the result equals the one of a context that
    grew its workspace on demand."""
    spec = [(RELU, 5, 33), (TANH, 33, 70), (LIN, 70, 3)]       # not the fused three-layer shape
    model = mk(mrl, spec)
    g = torch.Generator(device="cuda").manual_seed(5)
    p = torch.randn(model.PARAM_SIZE, device="cuda", generator=g) * 0.3
    x = torch.randn(300 * 5, device="cuda", generator=g)
    grown, reserved = mrl.DeviceContext("cuda:0"), mrl.DeviceContext("cuda:0")
    assert grown.workspace() == (0, 0)
    out_a = torch.zeros(300 * 3, device="cuda")
    model.forward_gpu_no_cache_ws(grown, out_a, x, p)
    grown.synchronize()
    need = grown.workspace()[0]
    assert need >= 2 * 300 * 70
    reserved.reserve(mlp_floats=need, rollout_floats=1000)
    assert reserved.workspace() == (need, 1000)
    reserved.reserve(mlp_floats=1, rollout_floats=0)              # never shrinks, 0 leaves as is
    assert reserved.workspace() == (need, 1000)
    out_b = torch.zeros(300 * 3, device="cuda")
    before = torch.cuda.memory_allocated()
    model.forward_gpu_no_cache_ws(reserved, out_b, x, p)
    reserved.synchronize()
    assert reserved.workspace() == (need, 1000) and torch.cuda.memory_allocated() == before
    assert torch.equal(out_a, out_b)
