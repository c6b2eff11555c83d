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


def _pair(mrl, ctx, N, T, hidden, kind, env="lunar"):
    E = {"lunar": mrl.LunarLanderV2, "lunarc": mrl.LunarLanderV2Continuous, "cartpole": mrl.CartPoleEnv,
         "pendulum": mrl.PendulumV2}[env]
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    head = mrl.StochasticActor(hidden, E.ACTION_DIM) if E.ACTION_DIM else mrl.Linear(hidden, E.NUM_ACTIONS)
    actor = mrl.seq(lin(E.OBS_DIM, hidden), lin(hidden, hidden), head)
    critic = mrl.seq(lin(E.OBS_DIM, hidden), lin(hidden, hidden), mrl.Linear(hidden, 1))
    g = torch.Generator(device="cuda").manual_seed(5)
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    out = []
    for _ in range(2):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = ap, cp
        E.reset_kernel_gpu(ctx, rb.states, 3)
        # some episodes end inside the range, so that in-place resets and the accounting are covered
        rows = rb.states.view(N, E.STATE_SIZE)
        if env in ("lunar", "lunarc"):
            rows[::3, 188] = 995.0    # step counter close to the limit
        elif env == "cartpole":
            rows[::3, 0] = 2.39       # cart next to the edge of the track, moving outwards
            rows[::3, 1] = 2.0
        else:
            rows[::3, 4] = 197.0      # step counter close to the limit
        rb.obs.copy_(rows[:, :E.OBS_DIM].reshape(-1))
        out.append(rb)
    return out


@pytest.mark.parametrize("env,N,T,hidden,kind", [
    ("lunar", 8192, 12, 256, "relu"), ("lunar", 1000, 9, 256, "tanh"), ("lunar", 77, 5, 256, "relu"),
    ("lunar", 300, 6, 64, "relu"),            # not fusable: the loop of single steps behind the same call
    ("cartpole", 8192, 12, 64, "relu"), ("cartpole", 77, 7, 64, "tanh"),
    ("pendulum", 8192, 12, 64, "tanh"), ("pendulum", 1000, 9, 64, "relu"),
    ("cartpole", 300, 6, 256, "relu"),        # not fusable
    ("lunarc", 8192, 12, 256, "tanh"), ("lunarc", 77, 6, 256, "relu"), ("lunarc", 300, 6, 64, "tanh"),
])
def test_rollout_steps_equals_single_steps(mrl, ctx, env, N, T, hidden, kind):
    print("case", env, N, T, hidden, kind, flush=True)
    one, many = _pair(mrl, ctx, N, T, hidden, kind, env)
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
