"""CPU checks of the drop-in boundary: the built library loads and exports every function that
include/mrl.h declares, and the Python binding table covers the same set (no compute calls)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    text = open(os.path.join(ROOT, "include", "mrl.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mrl_[a-z_0-9]+)\s*\(", text)))


def test_header_functions_are_exported(mrl):
    lib = ctypes.CDLL(os.path.join(ROOT, "mojo-rl_amd", "libmrl_hip.so"))
    names = declared()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), "libmrl_hip.so does not export %s" % n


def test_binding_table_matches_header(mrl):
    assert sorted(mrl._lib.exported_names()) == declared()
    assert mrl._lib.lib()._mrl_missing == []
    assert mrl._lib.lib().mrl_version() >= 100


def test_descriptor_queries_run_without_gpu(mrl):
    actor = mrl.seq(mrl.LinearReLU(8, 256), mrl.LinearReLU(256, 256), mrl.Linear(256, 4))
    assert (actor.PARAM_SIZE, actor.CACHE_SIZE, actor.OUT_DIM) == (69124, 8 + 4 * 256, 4)
    critic = mrl.seq(mrl.LinearReLU(8, 256), mrl.LinearReLU(256, 256), mrl.Linear(256, 1))
    assert critic.PARAM_SIZE == 68353
    g = mrl.seq(mrl.LinearTanh(24, 256), mrl.LinearTanh(256, 256), mrl.StochasticActor(256, 4))
    assert (g.PARAM_SIZE, g.OUT_DIM) == (73224, 8)
    ss, od, na, ad = (ctypes.c_int() for _ in range(4))
    for env, want in ((mrl.CartPoleEnv, (4, 4, 2, 0)), (mrl.PendulumV2, (8, 3, 0, 1)),
                      (mrl.LunarLanderV2, (192, 8, 4, 0))):
        mrl._lib.call("mrl_env_dims", env.ENV_ID, ctypes.byref(ss), ctypes.byref(od), ctypes.byref(na), ctypes.byref(ad))
        assert (ss.value, od.value, na.value, ad.value) == want
        assert (env.STATE_SIZE, env.OBS_DIM) == want[:2]


def test_missing_library_is_loud(mrl, tmp_path, monkeypatch):
    monkeypatch.setattr(mrl._lib, "LIB_PATH", str(tmp_path / "nope.so"))
    try:
        mrl._lib.load()
    except mrl.MrlError as e:
        assert "no fallback" in str(e)
    else:
        raise AssertionError("a missing HIP library must raise")


def test_no_gpu_means_error_not_fallback(mrl):
    import torch
    if torch.cuda.is_available():
        return
    try:
        mrl.DeviceContext("cuda:0")
    except mrl.MrlError as e:
        assert "no CPU fallback" in str(e)
    else:
        raise AssertionError("DeviceContext must refuse to run without a GPU")
