"""mrl_rollout_steps (many collection steps per launch) against the same steps issued one by one."""
import importlib
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mrl():
    return importlib.import_module("mojo-rl_amd")


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def _pair(mrl, ctx, N, T, hidden, kind):
    E = mrl.LunarLanderV2
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    actor = mrl.seq(lin(8, hidden), lin(hidden, hidden), mrl.Linear(hidden, 4))
    critic = mrl.seq(lin(8, hidden), lin(hidden, hidden), mrl.Linear(hidden, 1))
    g = torch.Generator(device="cuda").manual_seed(5)
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    out = []
    for _ in range(2):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = ap, cp
        E.reset_kernel_gpu(ctx, rb.states, 3)
        # some episodes end inside the range, so that in-place resets and the accounting are covered
        rb.states.view(N, 192)[::3, 188] = 995.0
        rb.obs.copy_(rb.states.view(N, 192)[:, :8].reshape(-1))
        out.append(rb)
    return out


@pytest.mark.parametrize("N,T,hidden,kind", [(8192, 12, 256, "relu"), (1000, 9, 256, "tanh"), (77, 5, 256, "relu"),
                                             (300, 6, 64, "relu")])
def test_rollout_steps_equals_single_steps(mrl, ctx, N, T, hidden, kind):
    print("case", N, T, hidden, kind, flush=True)
    one, many = _pair(mrl, ctx, N, T, hidden, kind)
    s0, ss, r0, rs = 1234567, 2654435761 * N + 7919, 99, 0x9E3779B97F4A7C15
    d1, d2 = one.descriptor(), many.descriptor()
    for t in range(T):
        mrl.ppo.rollout_step(ctx, d1, t, s0 + t * ss, 0, r0 + t * rs)
    # two launches: the second continues from the state the first left in HBM
    k = T // 2
    mrl.ppo.rollout_steps(ctx, d2, 0, k, s0, ss, 0, 0, r0, rs)
    mrl.ppo.rollout_steps(ctx, d2, k, T - k, s0 + k * ss, ss, 0, 0, r0 + k * rs, rs)
    ctx.synchronize()
    for name in ("r_obs", "r_actions", "r_log_probs", "r_values", "r_rewards", "r_dones", "states", "obs",
                 "ep_return", "ep_length"):
        a, b = getattr(one, name), getattr(many, name)
        assert torch.equal(a, b), "%s differs in %d places" % (name, int((a != b).sum()))
    cnt = int(one.done_count.item())
    assert cnt == int(many.done_count.item()) and cnt > 0
    key = lambda rb: sorted(zip(rb.done_returns[:cnt].tolist(), rb.done_lengths[:cnt].tolist()))
    assert key(one) == key(many)
