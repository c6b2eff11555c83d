"""ctypes loader for the CPU parity oracle (liborc.so).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg.  The shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liborc.so")

f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")
u32p = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")


class Layout(C.Structure):
    _fields_ = [(n, C.c_int) for n in (
        "num_bodies", "max_contacts", "max_joints", "max_edges", "obs_dim", "meta_size",
        "num_shapes", "bodies_off", "forces_off", "joints_off", "joint_count_off", "edges_off",
        "edge_count_off", "meta_off", "state_size")]


class Layer(C.Structure):
    _fields_ = [("kind", C.c_int), ("in_dim", C.c_int), ("out_dim", C.c_int)]


class Rms(C.Structure):
    _fields_ = [("count", C.c_double), ("mean", C.c_double), ("var_sum", C.c_double)]


LINEAR, LINEAR_RELU, LINEAR_TANH, STOCHASTIC_ACTOR = 0, 1, 2, 3


def build(force=False):
    """Compile liborc.so with the Makefile next to this file."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-s", "-C", _HERE, "liborc.so"])
    return _SO


def load():
    if not os.path.exists(_SO):
        build()
    lib = C.CDLL(_SO)
    LP = C.POINTER(Layout)
    YP = C.POINTER(Layer)
    sig = {
        "orc_xorshift32": (C.c_uint32, [C.c_uint32]),
        "orc_philox4x32_10": (None, [u32p, u32p, u32p]),
        "orc_philox_uniform4": (None, [C.c_uint64, C.c_uint64, C.c_uint64, f32p]),
        "orc_cartpole_step_batch": (None, [f32p, i32p, f32p, f32p, f32p, f32p, C.c_int]),
        "orc_cartpole_reset_batch": (None, [f32p, i32p, C.c_int, C.c_uint32]),
        "orc_cartpole_selective_reset_batch": (None, [f32p, i32p, f32p, C.c_int, C.c_uint32]),
        "orc_pendulum_step_batch": (None, [f32p, f32p, f32p, f32p, f32p, C.c_int]),
        "orc_pendulum_reset_batch": (None, [f32p, C.c_int, C.c_uint64]),
        "orc_pendulum_selective_reset_batch": (None, [f32p, f32p, C.c_int, C.c_uint64]),
        "orc_layout_make": (None, [LP] + [C.c_int] * 7),
        "orc_integrate_velocities": (None, [LP, f32p, C.c_float, C.c_float, C.c_float]),
        "orc_integrate_positions": (None, [LP, f32p, C.c_float]),
        "orc_edge_detect": (C.c_int, [LP, f32p, f32p, f32p]),
        "orc_flat_detect": (C.c_int, [LP, f32p, f32p, C.c_float, f32p]),
        "orc_contact_solve_velocity": (None, [LP, f32p, f32p, C.c_int, C.c_float, C.c_float]),
        "orc_contact_solve_position": (None, [LP, f32p, f32p, C.c_int, C.c_float, C.c_float]),
        "orc_joint_solve_velocity": (None, [LP, f32p, C.c_float]),
        "orc_joint_solve_position": (None, [LP, f32p, C.c_float, C.c_float]),
        "orc_lidar_ray": (C.c_float, [LP, f32p, C.c_float, C.c_float, C.c_float, C.c_float]),
        "orc_set_terrain_from_heights": (None, [LP, f32p, f32p, C.c_int, C.c_double, C.c_double]),
        "orc_ll_layout": (None, [LP]),
        "orc_ll_shapes": (None, [f32p]),
        "orc_ll_combined_seed": (C.c_uint64, [C.c_uint64, C.c_int]),
        "orc_ll_reset": (None, [f32p, C.c_uint64]),
        "orc_ll_set_wind": (None, [C.c_int, C.c_double, C.c_double]),
        "orc_ll_step": (None, [f32p, C.c_int, C.c_int, f32p, f32p, C.c_void_p, C.c_void_p]),
        "orc_ll_step_continuous": (None, [f32p, C.c_int, C.c_float, C.c_float, f32p, f32p, C.c_void_p, C.c_void_p]),
        "orc_ll_step_continuous_batch": (None, [f32p, f32p, f32p, f32p, f32p, C.c_int]),
        "orc_ll_reset_batch": (None, [f32p, C.c_int, C.c_uint64]),
        "orc_ll_selective_reset_batch": (None, [f32p, f32p, C.c_int, C.c_uint64]),
        "orc_ll_step_batch": (None, [f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int]),
        "orc_bw_layout": (None, [LP]),
        "orc_bw_shapes": (None, [f32p]),
        "orc_bw_reset": (None, [f32p, C.c_uint64]),
        "orc_bw_step": (None, [f32p, f32p, f32p, f32p]),
        "orc_bw_reset_batch": (None, [f32p, C.c_void_p, C.c_int, C.c_uint64]),
        "orc_bw_step_batch": (None, [f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int]),
        "orc_hc_layout": (None, [LP]),
        "orc_hc_shapes": (None, [f32p]),
        "orc_hc_reset": (None, [f32p, C.c_uint64]),
        "orc_hc_step": (None, [f32p, f32p, f32p, f32p]),
        "orc_hc_reset_batch": (None, [f32p, C.c_void_p, C.c_int, C.c_uint64]),
        "orc_hc_step_batch": (None, [f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int]),
        "orc_cr_tile_at": (C.c_int, [f32p, C.c_float, C.c_float, C.c_int]),
        "orc_cr_combined_seed": (C.c_uint64, [C.c_uint64, C.c_int]),
        "orc_cr_reset": (None, [f32p, C.c_uint64]),
        "orc_cr_step": (None, [f32p, f32p, f32p, f32p]),
        "orc_cr_set_step_form": (None, [C.c_int]),
        "orc_cr_reset_batch": (None, [f32p, C.c_void_p, C.c_int, C.c_uint64]),
        "orc_cr_step_batch": (None, [f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int]),
        "orc_planar_state_size": (C.c_int, [C.c_int]),
        "orc_planar_reset": (None, [C.c_int, f32p, C.c_uint64]),
        "orc_planar_step": (None, [C.c_int, f32p, f32p, f32p, f32p]),
        "orc_planar_reset_batch": (None, [C.c_int, f32p, C.c_void_p, C.c_int, C.c_uint64]),
        "orc_planar_step_batch": (None, [C.c_int, f32p, f32p, f32p, f32p, f32p, C.c_int, C.c_int]),
        "orc_mlp_param_size": (C.c_int, [YP, C.c_int]),
        "orc_mlp_cache_size": (C.c_int, [YP, C.c_int]),
        "orc_mlp_forward": (None, [YP, C.c_int, C.c_int, f32p, f32p, f32p, C.c_void_p]),
        "orc_mlp_backward": (None, [YP, C.c_int, C.c_int, f32p, f32p, f32p, f32p, C.c_void_p]),
        "orc_sample_categorical": (None, [f32p, C.c_int, C.c_int, C.c_uint32, f32p, f32p]),
        "orc_sample_gaussian": (None, [f32p, C.c_int, C.c_int, C.c_uint64, f32p, f32p]),
        "orc_add_obs_noise": (None, [f32p, C.c_int, C.c_int, C.c_float, C.c_uint32]),
        "orc_gae": (None, [C.c_int, C.c_int, f32p, f32p, f32p, f32p, C.c_double, C.c_double,
                           f32p, f32p]),
        "orc_normalize_advantages": (None, [f32p, C.c_int]),
        "orc_normalize_minibatch_host": (None, [f32p, C.c_int]),
        "orc_normalize_minibatch_fused": (None, [f32p, C.c_int]),
        "orc_ppo_actor_grad_discrete": (None, [f32p, f32p, f32p, f32p, C.c_int, C.c_int,
                                               C.c_float, C.c_float, f32p, f32p]),
        "orc_ppo_actor_grad_gaussian": (None, [f32p, f32p, f32p, f32p, C.c_int, C.c_int,
                                               C.c_float, C.c_float, f32p, f32p]),
        "orc_ppo_critic_grad": (None, [f32p, f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_float,
                                       C.c_float, f32p]),
        "orc_clip_grad_norm": (C.c_float, [f32p, C.c_int, C.c_float]),
        "orc_adam_step": (None, [f32p, f32p, f32p, C.c_int, C.c_int, C.c_double, C.c_double,
                                 C.c_double, C.c_double]),
        "orc_clamp_log_std": (None, [f32p, C.c_int, C.c_int]),
        "orc_rms_update": (None, [C.POINTER(Rms), f32p, C.c_int]),
        "orc_rms_normalize": (None, [C.POINTER(Rms), f32p, C.c_int]),
        "orc_shuffle_indices": (None, [C.c_int, f64p, i32p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def layers(spec):
    """spec: list of (kind, in_dim, out_dim) -> ctypes array of Layer."""
    arr = (Layer * len(spec))()
    for i, (k, a, b) in enumerate(spec):
        arr[i].kind, arr[i].in_dim, arr[i].out_dim = k, a, b
    return arr


def ll_layout(lib):
    L = Layout()
    lib.orc_ll_layout(C.byref(L))
    return L


def make_layout(lib, nb, mc, mj, me, obs, meta, ns):
    L = Layout()
    lib.orc_layout_make(C.byref(L), nb, mc, mj, me, obs, meta, ns)
    return L
