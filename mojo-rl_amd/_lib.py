"""ctypes binding of libmrl_hip.so (the C ABI declared in include/mrl.h).

The HIP library is the only compute path: if it cannot be loaded this module raises, there
is no CPU or eager fallback.  torch is used for device memory and the stream only.
"""
import ctypes as C
import os

# torch first: streams and device memory come from torch, so the library must bind to the HIP
# runtime that torch has already loaded into the process (one runtime per process, first one wins).
import torch  # noqa: F401

HERE = os.path.dirname(os.path.abspath(__file__))
# MRL_HIP_LIB points at an alternative build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("MRL_HIP_LIB") or os.path.join(HERE, "libmrl_hip.so")

MAX_LAYERS = 8
LINEAR, LINEAR_RELU, LINEAR_TANH, STOCHASTIC_ACTOR = 0, 1, 2, 3
ENV_CARTPOLE, ENV_PENDULUM, ENV_LUNARLANDER, ENV_BIPEDAL, ENV_HALFCHEETAH = 0, 1, 2, 3, 4
ENV_LUNARLANDER_CONTINUOUS = 5
ENV_CARRACING = 6
ENV_HOPPER_PLANAR, ENV_WALKER2D_PLANAR = 7, 8


class Layer(C.Structure):
    _fields_ = [("kind", C.c_int32), ("in_dim", C.c_int32), ("out_dim", C.c_int32)]


class MlpDesc(C.Structure):
    _fields_ = [("n_layers", C.c_int32), ("layers", Layer * MAX_LAYERS)]


class Rollout(C.Structure):
    _fields_ = [
        ("env_id", C.c_int32), ("n_envs", C.c_int32), ("obs_dim", C.c_int32), ("num_actions", C.c_int32),
        ("states", C.c_void_p), ("obs", C.c_void_p),
        ("actor_params", C.c_void_p), ("critic_params", C.c_void_p),
        ("actor", MlpDesc), ("critic", MlpDesc),
        ("r_obs", C.c_void_p), ("r_actions", C.c_void_p), ("r_log_probs", C.c_void_p),
        ("r_values", C.c_void_p), ("r_rewards", C.c_void_p), ("r_dones", C.c_void_p),
        ("ep_return", C.c_void_p), ("ep_length", C.c_void_p),
        ("done_returns", C.c_void_p), ("done_lengths", C.c_void_p),
        ("done_count", C.c_void_p), ("done_cap", C.c_int32),
    ]


class Update(C.Structure):
    _fields_ = (
        [(n, C.c_int32) for n in ("minibatch", "obs_dim", "act_width", "continuous")]
        + [("actor", MlpDesc), ("critic", MlpDesc)]
        + [(n, C.c_void_p) for n in (
            "actor_params", "critic_params", "actor_grads", "critic_grads", "actor_state", "critic_state",
            "r_obs", "r_actions", "r_log_probs", "r_values", "advantages", "returns",
            "mb_obs", "mb_actions", "mb_adv", "mb_ret", "mb_logp", "mb_val",
            "actor_out", "values", "g_actor_out", "g_values", "kl", "actor_cache", "critic_cache", "kl_flag")]
        + [(n, C.c_float) for n in ("clip_epsilon", "entropy_coef", "value_loss_coef", "max_grad_norm", "target_kl")]
        + [(n, C.c_int32) for n in ("clip_value", "norm_adv_per_minibatch")]
        + [(n, C.c_double) for n in ("actor_lr", "critic_lr", "beta1", "beta2", "eps")]
    )


class MrlError(RuntimeError):
    pass


P, I, U32, U64, F, D = C.c_void_p, C.c_int, C.c_uint32, C.c_uint64, C.c_float, C.c_double
DP, RP, UP = C.POINTER(MlpDesc), C.POINTER(Rollout), C.POINTER(Update)

# name -> argtypes; every function returns int (0 = ok) unless listed in _SPECIAL
SIGNATURES = {
    "mrl_ctx_create": [P, C.POINTER(P)],
    "mrl_ctx_destroy": [P],
    "mrl_ctx_synchronize": [P],
    "mrl_ctx_set_spin_limit": [P, C.c_uint],
    "mrl_ctx_workspace": [P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)],
    "mrl_ctx_reserve": [P, C.c_uint64, C.c_uint64],
    "mrl_profile_begin": [P, I],
    "mrl_profile_sample_every": [P, I],
    "mrl_profile_end": [P, I, C.POINTER(D), C.POINTER(I)],
    "mrl_env_dims": [I, C.POINTER(I), C.POINTER(I), C.POINTER(I), C.POINTER(I)],
    "mrl_env_reset": [P, I, I, P, U64],
    "mrl_env_selective_reset": [P, I, I, P, P, U64],
    "mrl_env_step": [P, I, I, P, P, P, P, P, U64],
    "mrl_env_step_autoreset": [P, I, I, P, P, P, P, P, U64, U64],
    "mrl_cartpole_bind_steps": [P, P, I, P],
    "mrl_lunar_set_wind": [P, I, D, D],
    "mrl_car_racing_set_step_form": [P, I],
    "mrl_mlp_param_size": [DP],
    "mrl_mlp_cache_size": [DP],
    "mrl_mlp_out_dim": [DP],
    "mrl_mlp_forward": [P, DP, I, P, P, P, P],
    "mrl_mlp_backward": [P, DP, I, P, P, P, P, P],
    "mrl_sample_categorical": [P, P, I, I, U32, P, P],
    "mrl_sample_gaussian": [P, P, I, I, U32, P, P],
    "mrl_greedy_actions": [P, P, I, I, I, P],
    "mrl_add_obs_noise": [P, P, I, I, F, U32],
    "mrl_gae": [P, I, I, P, P, P, P, D, D, P, P],
    "mrl_normalize_advantages": [P, P, I],
    "mrl_gather_minibatch": [P, P, I, I, I] + [P] * 12,
    "mrl_ppo_actor_grad_discrete": [P, P, P, P, P, I, I, F, F, P, P],
    "mrl_ppo_actor_grad_gaussian": [P, P, P, P, P, I, I, F, F, P, P],
    "mrl_ppo_critic_grad": [P, P, P, P, I, I, I, F, F, P],
    "mrl_clip_grad_norm": [P, P, I, F],
    "mrl_clip_grad_norm_static": [P, P, I, F],
    "mrl_adam_step": [P, P, P, P, I, I, D, D, D, D],
    "mrl_clamp_log_std": [P, P, I, I],
    "mrl_rms_update": [P, P, P, I],
    "mrl_rms_normalize": [P, P, P, I],
    "mrl_permutation": [P, P, I, U64],
    "mrl_permutation_from_uniforms": [P, P, I, P, P],
    "mrl_kl_check": [P, P, I, F, P],
    "mrl_init_uniform": [P, P, I, F, F, U64],
    "mrl_policy_step_discrete": [P, DP, DP, I, P, P, P, U32, P, P, P, P, P],
    "mrl_policy_step_gaussian": [P, DP, DP, I, P, P, P, U32, P, P, P, P, P],
    "mrl_rollout_step": [P, RP, I, U32, U64, U64],
    "mrl_rollout_steps": [P, RP, I, I, U32, U32, U64, U64, U64, U64],
    "mrl_rollout_fused": [RP],
    "mrl_ppo_update_minibatch": [P, UP, P, I, I],
    "mrl_ppo_update_epoch": [P, UP, P, I, I, I],
    "mrl_minibatch_adv_stats": [P, P, P, I, I, P],
}
_SPECIAL = {"mrl_version": (C.c_int, []), "mrl_last_error": (C.c_char_p, [])}
# size queries return a count, not a status
_RAW_INT = {"mrl_mlp_param_size", "mrl_mlp_cache_size", "mrl_mlp_out_dim", "mrl_rollout_fused"}


def exported_names():
    return list(SIGNATURES) + list(_SPECIAL)


def load():
    if not os.path.exists(LIB_PATH):
        raise MrlError(
            "libmrl_hip.so is not built (%s). Run `python -m __graft_entry__` or "
            "mojo-rl_amd/build.py; there is no fallback path." % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in _SPECIAL.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    missing = []
    for name, args in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            missing.append(name)
            continue
        fn.restype, fn.argtypes = C.c_int, args
    lib._mrl_missing = missing  # calling one of these raises; tests assert the list is empty
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = load()
    return _lib


def check(rc, what):
    if rc != 0:
        raise MrlError("%s failed (%d): %s" % (what, rc, lib().mrl_last_error().decode()))


def call(name, *args):
    if name in lib()._mrl_missing:
        raise MrlError("%s is not exported by %s" % (name, LIB_PATH))
    rc = getattr(lib(), name)(*args)
    if name in _RAW_INT:
        if rc < 0:
            check(rc, name)
        return rc
    check(rc, name)
    return rc


def make_desc(layers):
    """layers: sequence of (kind, in_dim, out_dim)."""
    if not 1 <= len(layers) <= MAX_LAYERS:
        raise MrlError("an MLP description holds 1..%d layers" % MAX_LAYERS)
    d = MlpDesc()
    d.n_layers = len(layers)
    for i, (k, a, b) in enumerate(layers):
        d.layers[i].kind, d.layers[i].in_dim, d.layers[i].out_dim = k, a, b
    return d
