"""Pins for the oracle's MLP layers and PPO utilities.

MLP: torch float64 autograd on the same weights.  GAE: O(T^2) direct evaluation.  Adam:
torch.optim.Adam and the reference's own first-step numbers.  PPO loss gradients: finite
differences of the scalar loss in float64; decision tables at the clip kinks.
"""
import ctypes as C
import math

import numpy as np
import torch

RELU, TANH, LIN, ACTOR = 1, 2, 0, 3


def torch_mlp(spec, params, x):
    off, h = 0, x
    for kind, i, o in spec:
        W = params[off:off + i * o].reshape(i, o); off += i * o
        b = params[off:off + o]; off += o
        y = h @ W + b
        if kind == RELU: h = torch.relu(y)
        elif kind == TANH: h = torch.tanh(y)
        elif kind == LIN: h = y
        else:
            ls = params[off:off + o]; off += o
            h = torch.cat([y, ls.clamp(-5, 2).expand(y.shape[0], o)], dim=1)
    return h


def run_case(orc, orcmod, spec, batch, seed):
    rng = np.random.default_rng(seed)
    ls = orcmod.layers(spec)
    P = orc.orc_mlp_param_size(ls, len(spec)); CSZ = orc.orc_mlp_cache_size(ls, len(spec))
    params = rng.uniform(-0.5, 0.5, P).astype(np.float32)
    x = rng.normal(size=(batch, spec[0][1])).astype(np.float32)
    od = spec[-1][2] * (2 if spec[-1][0] == ACTOR else 1)
    out = np.zeros((batch, od), np.float32); out_nc = np.zeros_like(out)
    cache = np.zeros(batch * CSZ, np.float32)
    orc.orc_mlp_forward(ls, len(spec), batch, x, params, out, cache.ctypes.data)
    orc.orc_mlp_forward(ls, len(spec), batch, x, params, out_nc, None)
    np.testing.assert_array_equal(out, out_nc)
    tp = torch.tensor(params, dtype=torch.float64, requires_grad=True)
    tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    ty = torch_mlp(spec, tp, tx)
    np.testing.assert_allclose(out, ty.detach().numpy(), rtol=2e-5, atol=2e-6)
    go = rng.normal(size=out.shape).astype(np.float32)
    ty.backward(torch.tensor(go, dtype=torch.float64))
    grads = np.zeros(P, np.float32); gin = np.zeros_like(x)
    orc.orc_mlp_backward(ls, len(spec), batch, go, params, cache, grads, gin.ctypes.data)
    np.testing.assert_allclose(grads, tp.grad.numpy(), rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(gin, tx.grad.numpy(), rtol=1e-4, atol=1e-5)
    # backward accumulates: a second call doubles the gradients
    orc.orc_mlp_backward(ls, len(spec), batch, go, params, cache, grads, None)
    np.testing.assert_allclose(grads, 2 * tp.grad.numpy(), rtol=1e-4, atol=2e-5)
    return cache, x, out


def test_mlp_against_torch_autograd(orc, orcmod):
    run_case(orc, orcmod, [(RELU, 8, 32), (RELU, 32, 32), (LIN, 32, 4)], 7, 0)
    run_case(orc, orcmod, [(TANH, 3, 16), (TANH, 16, 16), (ACTOR, 16, 2)], 5, 1)
    run_case(orc, orcmod, [(TANH, 5, 8), (LIN, 8, 1)], 9, 2)
    run_case(orc, orcmod, [(LIN, 4, 3)], 1, 3)


def test_cache_and_param_layout(orc, orcmod):
    spec = [(RELU, 3, 4), (TANH, 4, 5), (LIN, 5, 2)]
    cache, x, out = run_case(orc, orcmod, spec, 6, 4)
    ls = orcmod.layers(spec)
    assert orc.orc_mlp_param_size(ls, 3) == 3 * 4 + 4 + 4 * 5 + 5 + 5 * 2 + 2
    assert orc.orc_mlp_cache_size(ls, 3) == (3 + 4) + (4 + 5) + 5     # blocked per layer
    c0 = cache[:6 * 7].reshape(6, 7); c1 = cache[42:42 + 54].reshape(6, 9); c2 = cache[96:].reshape(6, 5)
    np.testing.assert_array_equal(c0[:, :3], x)                         # layer 0: [input | pre-activation]
    np.testing.assert_array_equal(c1[:, :4], np.maximum(c0[:, 3:], 0))  # layer 1 input = relu(pre-act)
    np.testing.assert_array_equal(c2, c1[:, 4:])                        # tanh layer caches its OUTPUT
    assert (np.abs(c1[:, 4:]) < 1).all()


def test_stochastic_actor_clamps_log_std(orc, orcmod):
    ls = orcmod.layers([(ACTOR, 2, 3)])
    params = np.array([0] * 6 + [1, 2, 3] + [-9.0, 0.25, 7.0], np.float32)
    out = np.zeros((1, 6), np.float32)
    orc.orc_mlp_forward(ls, 1, 1, np.zeros((1, 2), np.float32), params, out, None)
    np.testing.assert_array_equal(out[0], [1, 2, 3, -5.0, 0.25, 2.0])


def gae_direct(r, v, d, boot, g, lam):
    T = len(r)
    adv = np.zeros(T)
    vn = list(v[1:]) + [boot]
    delta = [r[t] + g * (0 if d[t] else vn[t]) - v[t] for t in range(T)]
    for t in range(T):
        acc, w = 0.0, 1.0
        for l in range(t, T):
            acc += w * delta[l]
            if d[l]:
                break
            w *= g * lam
        adv[t] = acc
    return adv


def test_gae_direct_sum(orc):
    rng = np.random.default_rng(5)
    T, N = 8, 6
    r = rng.normal(size=(T, N)).astype(np.float32); v = rng.normal(size=(T, N)).astype(np.float32)
    d = (rng.random((T, N)) < 0.25).astype(np.float32); boot = rng.normal(size=N).astype(np.float32)
    adv = np.zeros((T, N), np.float32); ret = np.zeros((T, N), np.float32)
    orc.orc_gae(T, N, r, v, d, boot, 0.99, 0.95, adv, ret)
    for e in range(N):
        want = gae_direct(r[:, e].astype(float), v[:, e].astype(float), d[:, e] > 0.5, float(boot[e]), 0.99, 0.95)
        np.testing.assert_allclose(adv[:, e], want, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(ret, adv + v, rtol=1e-6, atol=1e-6)


def test_normalisation_double_epsilon(orc):
    rng = np.random.default_rng(6)
    a = rng.normal(2.0, 3.0, 1000).astype(np.float32)
    for fn in (orc.orc_normalize_advantages, orc.orc_normalize_minibatch_host, orc.orc_normalize_minibatch_fused):
        x = a.copy(); fn(x, len(x))
        a64 = a.astype(np.float64)
        want = (a64 - a64.mean()) / (np.sqrt(a64.var() + 1e-8) + 1e-8)
        np.testing.assert_allclose(x, want, rtol=1e-4, atol=1e-5)
    x = np.full(16, 3.0, np.float32); orc.orc_normalize_advantages(x, 16)
    assert (x == 0).all()                                     # zero variance: eps keeps it finite


def test_adam_reference_first_step_and_torch(orc):
    # the reference's own self-check: g = 0.5 -> m = 0.05, v = 0.00025 after one step
    p = np.array([1.0], np.float32); st = np.zeros(2, np.float32)
    orc.orc_adam_step(p, np.array([0.5], np.float32), st, 1, 1, 0.001, 0.9, 0.999, 1e-8)
    np.testing.assert_allclose(st, [0.05, 0.00025], rtol=1e-6)
    assert abs(p[0] - (1.0 - 0.001)) < 1e-6
    rng = np.random.default_rng(7)
    p0 = rng.normal(size=50).astype(np.float32)
    p = p0.copy(); st = np.zeros(100, np.float32)
    tp = torch.tensor(p0, dtype=torch.float64, requires_grad=True)
    opt = torch.optim.Adam([tp], lr=3e-4, betas=(0.9, 0.999), eps=1e-8)
    for t in range(1, 4):
        g = rng.normal(size=50).astype(np.float32)
        orc.orc_adam_step(p, g, st, 50, t, 3e-4, 0.9, 0.999, 1e-8)
        tp.grad = torch.tensor(g, dtype=torch.float64); opt.step()
        np.testing.assert_allclose(p, tp.detach().numpy(), rtol=1e-5, atol=1e-6)
    assert st.reshape(50, 2)[:, 1].min() >= 0                  # interleaved (m, v) per parameter


def test_clip_grad_norm(orc):
    g = np.array([3.0, 4.0, 12.0], np.float32)                # norm 13
    s = orc.orc_clip_grad_norm(g, 3, 0.5)
    assert abs(s - 0.5 / (13 + 1e-8)) < 1e-7 and abs(np.linalg.norm(g) - 0.5) < 1e-6
    g = np.array([0.1, 0.2], np.float32); s = orc.orc_clip_grad_norm(g, 2, 0.5)
    assert s == 1.0 and list(g) == [np.float32(0.1), np.float32(0.2)]


def test_actor_grad_discrete_finite_difference(orc):
    rng = np.random.default_rng(8)
    mb, A = 6, 4
    logits = rng.normal(size=(mb, A)).astype(np.float32)
    acts = rng.integers(0, A, mb).astype(np.float32); adv = rng.normal(size=mb).astype(np.float32)
    p = torch.softmax(torch.tensor(logits, dtype=torch.float64), 1).numpy()
    old = (np.log(p[np.arange(mb), acts.astype(int)] + 1e-8) + rng.uniform(-0.1, 0.1, mb)).astype(np.float32)
    g0 = np.zeros((mb, A), np.float32); g = np.zeros((mb, A), np.float32); kl = np.zeros(mb, np.float32)
    orc.orc_ppo_actor_grad_discrete(logits, old, adv, acts, mb, A, 0.2, 0.0, g0, kl)
    orc.orc_ppo_actor_grad_discrete(logits, old, adv, acts, mb, A, 0.2, 0.01, g, kl)
    for b in range(mb):
        # surrogate term: autograd of -A * exp(log p_a - old) / MB w.r.t. the logits
        tl = torch.tensor(logits[b], dtype=torch.float64, requires_grad=True)
        lp = torch.log(torch.softmax(tl, 0)[int(acts[b])] + 1e-8)
        (-float(adv[b]) * torch.exp(lp - float(old[b])) / mb).backward()
        np.testing.assert_allclose(g0[b], tl.grad.numpy(), rtol=1e-4, atol=1e-6)
        # entropy term: the reference uses p * dH/dp (p held independent), not the softmax chain rule
        tp = torch.tensor(p[b], dtype=torch.float64, requires_grad=True)
        (-(tp * torch.log(tp + 1e-8)).sum()).backward()
        np.testing.assert_allclose(g[b] - g0[b], -0.01 * p[b] * tp.grad.numpy() / mb, rtol=2e-3, atol=1e-6)
        assert abs(kl[b] - (old[b] - math.log(p[b, int(acts[b])] + 1e-8))) < 1e-5   # signed old - new
    # clip kink: ratio outside [1-eps, 1+eps] zeroes the whole row whatever the advantage sign
    old2 = old.copy(); old2[0] -= 1.0; old2[1] += 1.0
    orc.orc_ppo_actor_grad_discrete(logits, old2, adv, acts, mb, A, 0.2, 0.01, g, kl)
    assert (g[0] == 0).all() and (g[1] == 0).all() and (g[2] != 0).any()


def test_sample_categorical(orc):
    rng = np.random.default_rng(9)
    n, A = 4000, 4
    logits = np.tile(np.array([0.0, 1.0, -1.0, 0.5], np.float32), (n, 1))
    a = np.zeros(n, np.float32); lp = np.zeros(n, np.float32)
    orc.orc_sample_categorical(logits, n, A, 1234, a, lp)
    p = np.exp(logits[0]) / np.exp(logits[0]).sum()
    freq = np.bincount(a.astype(int), minlength=A) / n
    assert np.abs(freq - p).max() < 0.03
    np.testing.assert_allclose(lp, np.log(p[a.astype(int)] + 1e-8), rtol=1e-5)
    # independent evaluation of the per-env stream for env 5
    M = 0xFFFFFFFF

    def xs(x):
        x ^= (x << 13) & M; x ^= x >> 17; x ^= (x << 5) & M
        return x
    u = np.float32(xs(xs(1234 ^ ((5 * 2654435761) & M)))) / np.float32(M)
    want = int(np.searchsorted(np.cumsum(p.astype(np.float32)), u, side="right"))
    assert int(a[5]) == min(want, A - 1)


def test_sample_gaussian(orc):
    n, A = 20000, 2
    out = np.tile(np.array([0.5, -1.0, -0.5, 0.3], np.float32), (n, 1))   # mean | log_std
    a = np.zeros((n, A), np.float32); lp = np.zeros(n, np.float32)
    orc.orc_sample_gaussian(out, n, A, 99, a, lp)
    std = np.exp(np.array([-0.5, 0.3]))
    assert np.abs(a.mean(0) - [0.5, -1.0]).max() < 0.03 and np.abs(a.std(0) / std - 1).max() < 0.03
    z = (a - [0.5, -1.0]) / (std + 1e-6)
    want = (-0.5 * (math.log(2 * math.pi) + 2 * np.array([-0.5, 0.3]) + z * z)).sum(1)
    np.testing.assert_allclose(lp, want, rtol=1e-4, atol=1e-4)


def test_add_obs_noise(orc):
    """kernels.mojo:882-925: obs += std * z, z from Philox(seed + i * OBS + d) by Box-Muller -- the
    standard normal that the Gaussian sampler draws for (mean 0, log_std 0) on the same stream."""
    n, D = 5000, 8
    obs0 = np.random.default_rng(1).normal(size=(n, D)).astype(np.float32)
    obs = obs0.copy()
    orc.orc_add_obs_noise(obs, n, D, 0.25, 77)
    z = (obs.astype(np.float64) - obs0) / 0.25
    assert abs(z.mean()) < 0.02 and abs(z.std() - 1.0) < 0.02
    assert abs(np.mean(z ** 3)) < 0.05 and abs(np.mean(z ** 4) - 3.0) < 0.15        # Gaussian, not just unit variance
    assert abs(np.corrcoef(z[:, 0], z[:, 1])[0, 1]) < 0.05                           # entries are independent
    # the very numbers of the sampler's noise for the same streams
    out = np.zeros((n, 2 * D), np.float32)
    a, lp = np.zeros((n, D), np.float32), np.zeros(n, np.float32)
    orc.orc_sample_gaussian(out, n, D, 77, a, lp)
    zero = np.zeros((n, D), np.float32)
    orc.orc_add_obs_noise(zero, n, D, 1.0, 77)
    np.testing.assert_array_equal(zero, a)
    # Box-Muller from the oracle's own uniforms, in float64
    u = np.zeros(4, np.float32)
    orc.orc_philox_uniform4(77 + 3 * D + 5, 0, 0, u)
    want = math.sqrt(-2.0 * math.log(float(u[0]) + 1e-8)) * math.cos(2 * math.pi * float(u[1]))
    assert abs(zero[3, 5] - want) < 1e-5
    # std <= 0 leaves the observations alone; the same seed gives the same noise
    same = obs0.copy(); orc.orc_add_obs_noise(same, n, D, 0.0, 77)
    np.testing.assert_array_equal(same, obs0)
    again = obs0.copy(); orc.orc_add_obs_noise(again, n, D, 0.25, 77)
    np.testing.assert_array_equal(again, obs)


def test_actor_grad_gaussian_finite_difference(orc):
    rng = np.random.default_rng(10)
    mb, A = 5, 3
    out = np.concatenate([rng.normal(size=(mb, A)), rng.uniform(-1, 0.5, (mb, A))], 1).astype(np.float32)
    acts = (out[:, :A] + rng.normal(size=(mb, A)) * 0.5).astype(np.float32)
    adv = rng.normal(size=mb).astype(np.float32)

    def logp(o, a):
        mean, ls = o[:A], o[A:]
        z = (a - mean) / (torch.exp(ls) + 1e-6)
        return (-0.5 * (math.log(2 * math.pi) + 2 * ls + z * z)).sum()
    old = np.array([float(logp(torch.tensor(out[b], dtype=torch.float64), torch.tensor(acts[b], dtype=torch.float64)))
                    for b in range(mb)], np.float32) + rng.uniform(-0.05, 0.05, mb).astype(np.float32)
    g = np.zeros((mb, 2 * A), np.float32); kl = np.zeros(mb, np.float32)
    orc.orc_ppo_actor_grad_gaussian(out, old, adv, acts, mb, A, 0.2, 0.01, g, kl)
    for b in range(mb):
        to = torch.tensor(out[b], dtype=torch.float64, requires_grad=True)
        lp = logp(to, torch.tensor(acts[b], dtype=torch.float64))
        ratio = torch.exp(lp - float(old[b]))
        ent = (0.5 * (math.log(2 * math.pi) + 1 + 2 * to[A:])).sum()
        ((-float(adv[b]) * ratio - 0.01 * ent) / mb).backward()
        # the kernel's d/dlog_std treats (std + 1e-6) as std: agreement to ~1e-5 relative
        np.testing.assert_allclose(g[b], to.grad.numpy(), rtol=2e-4, atol=2e-6)
        r = float(ratio.detach()); assert abs(kl[b] - max(0.0, (r - 1) - math.log(r))) < 1e-5
    # clipped iff clip(ratio)*A < ratio*A: ratio high & A>0, or ratio low & A<0
    old2 = old.copy(); old2[:] = old - 1.0
    adv2 = np.array([1, -1, 1, -1, 1], np.float32)
    orc.orc_ppo_actor_grad_gaussian(out, old2, adv2, acts, mb, A, 0.2, 0.01, g, kl)
    assert (g[0] == 0).all() and (g[1] != 0).any() and (g[2] == 0).all() and (g[3] != 0).any()


def test_critic_grad_conventions(orc):
    v = np.array([1.0, 1.0, 1.0, 0.0], np.float32); vo = np.array([0.95, 0.5, 0.5, 0.5], np.float32)
    ret = np.array([2.0, 2.0, 0.0, 0.4], np.float32); g = np.zeros(4, np.float32)
    orc.orc_ppo_critic_grad(v, vo, ret, 4, 0, 0, 0.5, 0.2, g)            # discrete: 2 c_v (V - R) / MB
    np.testing.assert_allclose(g, 2 * 0.5 * (v - ret) / 4, rtol=1e-6)
    orc.orc_ppo_critic_grad(v, vo, ret, 4, 1, 0, 0.5, 0.2, g)            # continuous: (V - R) / MB
    np.testing.assert_allclose(g, (v - ret) / 4, rtol=1e-6)
    # clipped variants vs autograd of max((V-R)^2, (clip(V)-R)^2) (times c_v, or times 1/2)
    for conv, scale in ((0, 0.5), (1, 0.5)):
        orc.orc_ppo_critic_grad(v, vo, ret, 4, conv, 1, 0.5, 0.2, g)
        tv = torch.tensor(v, dtype=torch.float64, requires_grad=True)
        tvo, tr = torch.tensor(vo, dtype=torch.float64), torch.tensor(ret, dtype=torch.float64)
        vc = tvo + (tv - tvo).clamp(-0.2, 0.2)
        (scale * torch.maximum((tv - tr) ** 2, (vc - tr) ** 2) / 4).sum().backward()
        np.testing.assert_allclose(g, tv.grad.numpy(), rtol=1e-5, atol=1e-7)


def test_running_mean_std_chan_merge(orc, orcmod):
    rng = np.random.default_rng(11)
    a = rng.normal(1, 2, 300).astype(np.float32); b = rng.normal(-3, 0.5, 200).astype(np.float32)
    r = orcmod.Rms(0, 0, 0)
    orc.orc_rms_update(C.byref(r), a, 300); orc.orc_rms_update(C.byref(r), b, 200)
    allv = np.concatenate([a, b]).astype(np.float64)
    assert abs(r.mean - allv.mean()) < 1e-9 and abs(r.var_sum / r.count - allv.var()) < 1e-9
    x = a.copy(); orc.orc_rms_normalize(C.byref(r), x, 300)
    np.testing.assert_allclose(x, (a - allv.mean()) / (math.sqrt(allv.var() + 1e-8) + 1e-8), rtol=1e-5, atol=1e-6)
    r0 = orcmod.Rms(1, 5.0, 0); y = np.array([6.0], np.float32); orc.orc_rms_normalize(C.byref(r0), y, 1)
    assert abs(y[0] - 1.0) < 1e-6                                         # variance defaults to 1 while count < 2


def test_shuffle_indices_brute_force(orc):
    """orc_shuffle_indices (core/utils/shuffle.mojo:21-48) pinned without retyping its loop:
    (i) over an exhaustive grid of draws for n <= 5 -- one draw per bin of every iteration, at the
    bin's lower edge, middle and just below its upper edge -- the result equals the product of the
    transposition MATRICES (i j_i) applied to the identity vector in loop order (n-1 first), and
    the n! bin choices give n! different permutations (Fisher-Yates is a bijection from bin
    choices to permutations: a dropped iteration, an off-by-one in the range or a bin computed
    from i instead of i + 1 breaks this count); (ii) u = 1.0 falls back to j = i (no move) and
    u = 0.0 swaps with position 0; (iii) draws are consumed in loop order, u[0] by i = n - 1."""
    import itertools
    for n in range(1, 6):
        seen = set()
        bins = [range(i + 1) for i in range(n - 1, 0, -1)]          # iteration i = n-1 .. 1
        for choice in itertools.product(*bins):
            mats = np.eye(n, dtype=np.int64)
            for i, j in zip(range(n - 1, 0, -1), choice):
                t = np.eye(n, dtype=np.int64)
                t[[i, j]] = t[[j, i]]
                mats = t @ mats
            want = (mats @ np.arange(n)).astype(np.int32)
            for frac in (0.0, 0.5, 1.0 - 1e-9):
                u = np.array([(j + frac) / (i + 1) for i, j in zip(range(n - 1, 0, -1), choice)] + [0.0],
                             np.float64)
                got = np.full(n, -1, np.int32)
                orc.orc_shuffle_indices(n, u, got)
                np.testing.assert_array_equal(got, want)
            seen.add(tuple(want.tolist()))
        assert len(seen) == math.factorial(n)
    got = np.zeros(4, np.int32)
    orc.orc_shuffle_indices(4, np.array([1.0, 1.0, 1.0]), got)
    np.testing.assert_array_equal(got, [0, 1, 2, 3])
    orc.orc_shuffle_indices(4, np.array([0.0, 0.0, 0.0]), got)
    np.testing.assert_array_equal(got, [1, 2, 3, 0])           # 0<->3, then 3(at 0)<->2 ..., a rotation
    orc.orc_shuffle_indices(4, np.array([0.0, 0.99, 0.99]), got)    # only the first draw (i = 3) moves anything
    np.testing.assert_array_equal(got, [3, 1, 2, 0])
