"""Host-side mirror of the reference interfaces: what can be checked without a GPU.

Sizes come from the library's host-only queries (mrl_mlp_param_size, mrl_env_dims ...), so
these tests also show that the C ABI loads and answers on a machine with no device."""
import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_param_counts_of_the_five_configs(mrl):
    def nets(obs, hidden, out, relu, gauss):
        Lay = mrl.LinearReLU if relu else mrl.LinearTanh
        head = mrl.StochasticActor(hidden, out) if gauss else mrl.Linear(hidden, out)
        actor = mrl.seq(Lay(obs, hidden), Lay(hidden, hidden), head)
        critic = mrl.seq(Lay(obs, hidden), Lay(hidden, hidden), mrl.Linear(hidden, 1))
        return actor, critic
    # parameter counts of the reference's agents for the five benchmark configurations
    for obs, hidden, out, relu, gauss, pa, pc in ((4, 64, 2, True, False, 4610, 4545),
                                                  (3, 64, 1, False, True, 4482, 4481),
                                                  (8, 256, 4, True, False, 69124, 68353),
                                                  (24, 256, 4, False, True, 73224, 72449),
                                                  (17, 256, 6, False, True, 71948, 70657)):
        a, c = nets(obs, hidden, out, relu, gauss)
        assert (a.PARAM_SIZE, c.PARAM_SIZE) == (pa, pc)
        assert a.IN_DIM == obs and c.OUT_DIM == 1
        assert a.OUT_DIM == (2 * out if gauss else out)
        # cache of the two hidden layers: input + (pre-activation or tanh output) per layer, then the
        # head's input (deep_agents/ppo/ppo.mojo:779-780: OBS + 4 * HIDDEN)
        assert a.CACHE_SIZE == obs + 4 * hidden and c.CACHE_SIZE == obs + 4 * hidden
        assert a.WORKSPACE_SIZE_PER_SAMPLE == 2 * hidden


def test_seq_flattens_nested_models(mrl):
    inner = mrl.seq(mrl.LinearReLU(8, 16), mrl.LinearReLU(16, 16))
    m = mrl.seq(inner, mrl.Linear(16, 3))
    assert [l[0] for l in m.layers] == [mrl.LINEAR_RELU, mrl.LINEAR_RELU, mrl.LINEAR]
    assert m.PARAM_SIZE == 8 * 16 + 16 + 16 * 16 + 16 + 16 * 3 + 3


def test_bad_descriptions_raise(mrl):
    with pytest.raises(mrl.MrlError):
        mrl.Model([])
    with pytest.raises(mrl.MrlError):
        mrl.Model([(mrl.LINEAR, 4, 4)] * 9)
    with pytest.raises(mrl.MrlError):                 # dims of adjacent layers do not chain
        mrl.seq(mrl.Linear(4, 8), mrl.Linear(7, 2))
    with pytest.raises(mrl.MrlError):                 # the actor head must be last
        mrl.seq(mrl.StochasticActor(4, 2), mrl.Linear(4, 2))
    with pytest.raises(mrl.MrlError):
        mrl.Model([(17, 4, 4)])


def test_env_constants_match_the_library_and_the_oracle_layouts(mrl, orc, orcmod):
    want = {"CartPoleEnv": (4, 4, 2, 0), "PendulumV2": (8, 3, 0, 1), "LunarLanderV2": (192, 8, 4, 0),
            "LunarLanderV2Continuous": (192, 8, 0, 2), "BipedalWalkerV2": (950, 24, 0, 4),
            "HalfCheetahPlanarV2": (253, 17, 0, 6)}
    for name, (ss, od, na, ad) in want.items():
        E = getattr(mrl, name)
        assert (E.STATE_SIZE, E.OBS_DIM, E.NUM_ACTIONS, E.ACTION_DIM) == (ss, od, na, ad)
        vals = [ctypes.c_int() for _ in range(4)]
        mrl._lib.call("mrl_env_dims", E.ENV_ID, *[ctypes.byref(v) for v in vals])
        assert tuple(v.value for v in vals) == (ss, od, na, ad)
    for fn, ss in ((orc.orc_ll_layout, 192), (orc.orc_bw_layout, 950), (orc.orc_hc_layout, 253)):
        L = orcmod.Layout()
        fn(ctypes.byref(L))
        assert L.state_size == ss
    with pytest.raises(mrl.MrlError):
        mrl._lib.call("mrl_env_dims", 99, *[ctypes.byref(ctypes.c_int()) for _ in range(4)])


def test_null_context_is_an_error_not_a_crash(mrl):
    with pytest.raises(mrl.MrlError, match="ctx"):
        mrl._lib.call("mrl_gae", None, 1, 1, None, None, None, None, 0.99, 0.95, None, None)
    with pytest.raises(mrl.MrlError):
        mrl._lib.call("mrl_permutation", None, None, 10, 1)
    with pytest.raises(mrl.MrlError, match="ctx"):
        mrl._lib.call("mrl_greedy_actions", None, None, 4, 2, 0, None)
    with pytest.raises(mrl.MrlError, match="NULL"):
        mrl._lib.call("mrl_rollout_steps", None, None, 0, 1, 0, 0, 0, 0, 0, 0)
    assert b"" != mrl._lib.lib().mrl_last_error()


def test_adam_rejects_mismatched_buffers(mrl):
    import torch
    opt = mrl.Adam(lr=1e-3)
    with pytest.raises(mrl.MrlError):
        opt.step_gpu(None, torch.zeros(4), torch.zeros(3), torch.zeros(8))
    assert opt.t == 0


def test_bench_refuses_more_than_one_gpu():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert p.returncode != 0 and "one MI355X" in (p.stderr + p.stdout)
