#!/usr/bin/env python3
"""Headline benchmark: batched rollout (policy + value forward, sampling, env step with auto-reset,
rollout stores) and the PPO update, on one MI355X.

Default workload: LunarLander, 8192 envs, nets 8-256-256-4 / 8-256-256-1 (the north-star
configuration).  One "step" = one collection step over all envs.  `value` = env-steps/s including
the policy forward, inputs resident in HBM.  The PPO update throughput (samples/s) is reported
beside it in the same JSON line, with the roofline figures of the dominant kernel (device time
measured live with HIP events on the launch stream) and the CPU baseline (the oracle's C
restatement of the reference's CPU path, timed on this box's host cores on a bounded sample).
`--workload` selects one of the other benchmark configurations (parity-test cases otherwise).
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS, MFMA_FP32_PEAK_TFLOPS = 8000.0, 157.3

# name -> env class, envs, hidden width, hidden activation, algorithmic bytes per env-step (live
# fields of the reference row layout, each read once and written once), description
WORKLOADS = {
    "cartpole": ("CartPoleEnv", 4096, 64, "tanh", 60, "CartPole-v1 discrete, 4096 envs, nets 4-64-64-2 / 4-64-64-1 (tanh)"),
    "pendulum": ("PendulumV2", 16384, 64, "tanh", 72, "Pendulum continuous, 16384 envs, Gaussian 3-64-64-1 + value"),
    "lunarlander": ("LunarLanderV2", 8192, 256, "relu", 672,
                    "LunarLander-v2 discrete, 8192 envs, policy 8-256-256-4 + value 8-256-256-1 "
                    "(the north-star configuration)"),
    "bipedal": ("BipedalWalkerV2", 4096, 256, "tanh", 3964,
                "BipedalWalker continuous, 4096 envs, Gaussian 24-256-256-4 + value"),
    "halfcheetah": ("HalfCheetahPlanarV2", 4096, 256, "tanh", 1112,
                    "HalfCheetah planar continuous, 4096 envs, Gaussian 17-256-256-6 + value"),
    # per env-step: the 300 x 9 tile table read once (10800 B) + 40 floats of car state read and written
    "carracing": ("CarRacingV2", 4096, 256, "tanh", 11120,
                  "CarRacing (state-based) continuous, 4096 envs, Gaussian 13-256-256-3 + value"),
    # Float64 rows read and written once (248 / 392 B each way) + actions, observation, reward, done
    "hopper": ("HopperPlanar", 4096, 256, "tanh", 560,
               "HopperPlanar continuous (Float64 simplified physics), 4096 envs, Gaussian 11-256-256-3 + value"),
    "walker2d": ("Walker2dPlanar", 4096, 256, "tanh", 884,
                 "Walker2dPlanar continuous (Float64 simplified physics), 4096 envs, Gaussian 17-256-256-6 + value"),
}


def build_nets(mrl, E, hidden, act):
    lay = mrl.LinearReLU if act == "relu" else mrl.LinearTanh
    continuous = E.NUM_ACTIONS == 0
    head = mrl.StochasticActor(hidden, E.ACTION_DIM) if continuous else mrl.Linear(hidden, E.NUM_ACTIONS)
    actor = mrl.seq(lay(E.OBS_DIM, hidden), lay(hidden, hidden), head)
    critic = mrl.seq(lay(E.OBS_DIM, hidden), lay(hidden, hidden), mrl.Linear(hidden, 1))
    return actor, critic, continuous


def fwd_flops(E, hidden):
    a = E.ACTION_DIM if E.NUM_ACTIONS == 0 else E.NUM_ACTIONS
    return 2 * ((E.OBS_DIM * hidden + hidden * hidden + hidden * a) + (E.OBS_DIM * hidden + hidden * hidden + hidden))


def _cpu_rollout(np, orc, o, n_envs, steps, seed):
    """`steps` collection steps of `n_envs` LunarLander envs on the calling thread (the oracle's C
    restatement of the reference CPU path: actor / critic forward, sampling, env step, reset)."""
    OBS, HIDDEN, NA = 8, 256, 4
    la = orc.layers([(1, OBS, HIDDEN), (1, HIDDEN, HIDDEN), (0, HIDDEN, NA)])
    lc = orc.layers([(1, OBS, HIDDEN), (1, HIDDEN, HIDDEN), (0, HIDDEN, 1)])
    rng = np.random.default_rng(seed)
    pa = rng.uniform(-0.1, 0.1, o.orc_mlp_param_size(la, 3)).astype(np.float32)
    pc = rng.uniform(-0.1, 0.1, o.orc_mlp_param_size(lc, 3)).astype(np.float32)
    s = np.zeros((n_envs, 192), np.float32)
    o.orc_ll_reset_batch(s, n_envs, 1 + seed)
    obs = np.ascontiguousarray(s[:, :8])
    logits, values = np.zeros((n_envs, NA), np.float32), np.zeros((n_envs, 1), np.float32)
    a, lp = np.zeros(n_envs, np.float32), np.zeros(n_envs, np.float32)
    r, d = np.zeros(n_envs, np.float32), np.zeros(n_envs, np.float32)
    for t in range(steps):
        o.orc_mlp_forward(la, 3, n_envs, obs, pa, logits, None)
        o.orc_mlp_forward(lc, 3, n_envs, obs, pc, values, None)
        o.orc_sample_categorical(logits, n_envs, NA, 100 + t, a, lp)
        o.orc_ll_step_batch(s, a, r, d, obs, n_envs, 1)
        o.orc_ll_selective_reset_batch(s, d, n_envs, 500 + t)
        obs[:] = s[:, :8]


def _cpu_update(np, orc, o, mb, seed):
    """One PPO minibatch update of `mb` samples on the calling thread with the oracle's pieces in the
    reference's order: per-minibatch advantage normalisation, actor and critic forward with caches,
    loss gradients, backward, global-norm clip, Adam (north-star nets 8-256-256-4 and 8-256-256-1)."""
    OBS, HIDDEN, NA = 8, 256, 4
    la = orc.layers([(1, OBS, HIDDEN), (1, HIDDEN, HIDDEN), (0, HIDDEN, NA)])
    lc = orc.layers([(1, OBS, HIDDEN), (1, HIDDEN, HIDDEN), (0, HIDDEN, 1)])
    rng = np.random.default_rng(seed)
    pa = rng.uniform(-0.1, 0.1, o.orc_mlp_param_size(la, 3)).astype(np.float32)
    pc = rng.uniform(-0.1, 0.1, o.orc_mlp_param_size(lc, 3)).astype(np.float32)
    obs = rng.normal(size=(mb, OBS)).astype(np.float32)
    act = rng.integers(0, NA, mb).astype(np.float32)
    adv, ret = rng.normal(size=mb).astype(np.float32), rng.normal(size=mb).astype(np.float32)
    old_lp, old_v = np.full(mb, -1.3, np.float32), rng.normal(size=mb).astype(np.float32)
    o.orc_normalize_minibatch_host(adv, mb)
    for layers, params, lr in ((la, pa, 3e-4), (lc, pc, 1e-3)):
        actor = layers is la
        width = NA if actor else 1
        cache = np.zeros(mb * o.orc_mlp_cache_size(layers, 3), np.float32)
        out = np.zeros((mb, width), np.float32)
        o.orc_mlp_forward(layers, 3, mb, obs, params, out, cache.ctypes.data)
        g_out = np.zeros((mb, width), np.float32)
        if actor:
            kl = np.zeros(mb, np.float32)
            o.orc_ppo_actor_grad_discrete(out, old_lp, adv, act, mb, NA, 0.2, 0.01, g_out, kl)
        else:
            gv = np.zeros(mb, np.float32)
            o.orc_ppo_critic_grad(out.reshape(-1), old_v, ret, mb, 0, 1, 0.5, 0.2, gv)
            g_out[:, 0] = gv
        g = np.zeros(params.size, np.float32)
        o.orc_mlp_backward(layers, 3, mb, g_out, params, cache, g, None)
        o.orc_clip_grad_norm(g, g.size, 0.5)
        state = np.zeros(2 * g.size, np.float32)
        o.orc_adam_step(params, g, state, g.size, 1, lr, 0.9, 0.999, 1e-8)


def cpu_baseline(np, n_envs=2048, steps=120):
    """The CPU figures beside the GPU ones: the oracle timed on this box's host cores on a bounded
    sample of the default workload.  Rollout: once on every core of this job's CPU share (the envs
    split evenly over the threads, each thread its own rollout loop; the C calls release the GIL), and
    once on a single thread, which is how the reference's own CPU loop runs.  Update: minibatches of
    4096 on one thread (the reference's CPU trainer is a serial loop over samples and layers) and one
    minibatch per thread on all cores."""
    from concurrent.futures import ThreadPoolExecutor
    from oracle import orc
    o = orc.load()
    cores = max(1, min(int(os.environ.get("OMP_NUM_THREADS", "16")), os.cpu_count() or 1, 16))
    t0 = time.perf_counter()
    _cpu_rollout(np, orc, o, n_envs // 4, steps, 0)
    dt1 = time.perf_counter() - t0
    single = (n_envs // 4) * steps / dt1
    per = 4 * n_envs // cores
    t0 = time.perf_counter()
    with ThreadPoolExecutor(cores) as pool:
        list(pool.map(lambda k: _cpu_rollout(np, orc, o, per, steps, k), range(cores)))
    dtc = time.perf_counter() - t0
    mb = 4096
    t0 = time.perf_counter()
    _cpu_update(np, orc, o, mb, 0)
    du1 = time.perf_counter() - t0
    t0 = time.perf_counter()
    with ThreadPoolExecutor(cores) as pool:
        list(pool.map(lambda k: _cpu_update(np, orc, o, mb, k), range(cores)))
    duc = time.perf_counter() - t0
    return {"value": per * cores * steps / dtc, "unit": "env-steps/s", "cores": cores, "kind": "port",
            # cores = threads used: this job's CPU share of the box (OMP_NUM_THREADS there, at most 16);
            # host_cores = what the host reports, most of which belongs to other jobs
            "host_cores": os.cpu_count(),
            "single_thread_value": single,
            "update_samples_per_s": mb * cores / duc, "update_single_thread_samples_per_s": mb / du1,
            "sample": "LunarLander collection steps (env step + actor / critic forward + sampling + reset): "
                      "%d envs x %d steps on %d threads in %.1f s; %d envs x %d steps on one thread in %.1f s; "
                      "PPO update: %d minibatches of %d samples, one per thread, in %.1f s; one minibatch on one "
                      "thread in %.1f s" % (per * cores, steps, cores, dtc, n_envs // 4, steps, dt1, cores, mb, duc, du1)}


# batch at which the stand-alone env-step kernel is timed a second time: large enough that the chip is
# filled many times over, which is where its rate against the HBM roofline peaks
ENV_STEP_PEAK_BATCH = {"lunarlander": 524288, "bipedal": 65536, "halfcheetah": 131072, "carracing": 32768,
                       "cartpole": 4194304, "pendulum": 4194304, "hopper": 1048576, "walker2d": 1048576}


def env_step_at_large_batch(mrl, ctx, torch, E, workload, bytes_per_step, steps=40):
    """The stand-alone step + auto-reset kernel alone (actions fixed, no policy), HIP events around
    each launch on the launch stream, median launch: us per step, GB/s of algorithmic bytes, fraction
    of the HBM peak."""
    n = ENV_STEP_PEAK_BATCH[workload]
    s = torch.zeros(n * E.STATE_SIZE, device="cuda")
    E.reset_kernel_gpu(ctx, s, 1)
    if E.NUM_ACTIONS:
        a = torch.randint(0, E.NUM_ACTIONS, (n,), device="cuda").float()
    else:
        a = torch.rand(n * E.ACTION_DIM, device="cuda") * 2 - 1
    r, d, o = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda"), torch.zeros(n * E.OBS_DIM, device="cuda")
    for t in range(60):      # into the mix of flight, contacts and resets
        E.step_autoreset_kernel_gpu(ctx, s, a, r, d, o, t, 100 + t)
    ctx.synchronize()
    with torch.cuda.stream(ctx.stream):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2 * steps)]
        for t in range(steps):
            ev[2 * t].record(ctx.stream)
            E.step_autoreset_kernel_gpu(ctx, s, a, r, d, o, 200 + t, 1000 + t)
            ev[2 * t + 1].record(ctx.stream)
    ctx.synchronize()
    us = sorted(ev[2 * t].elapsed_time(ev[2 * t + 1]) * 1e3 for t in range(steps))
    med = us[len(us) // 2]
    gbs = bytes_per_step * n / (med * 1e-6) / 1e9
    return {"n_envs": n, "us_per_step": med, "env_steps_per_s": n / (med * 1e-6), "GBs": gbs,
            "frac_hbm": gbs / HBM_PEAK_GBS, "bytes_per_env_step": bytes_per_step}


def measured_traffic(steps_per_launch):
    """HBM bytes per launch by kernel name, from the committed counter summary
    (profiles/bench_lunarlander8192_hbm_traffic.md: FETCH_SIZE / WRITE_SIZE readings of
    rocprofv3 --pmc runs of this script, already scaled by the copy-kernel calibration).  A row of
    the fused collection kernel counts only for launches of the number of steps it was measured at.
    Empty when the file is absent."""
    path = os.path.join(ROOT, "profiles", "bench_lunarlander8192_hbm_traffic.md")
    out = {}
    if not os.path.exists(path):
        return out
    with open(path) as f:
        for line in f:
            cells = [c.strip() for c in line.strip().strip("|").split("|")]
            if len(cells) == 7 and cells[5].isdigit() and cells[1] in ("", str(steps_per_launch)):
                out[cells[0].replace("void ", "")] = int(cells[5])
    return out


EVENT_STRIDE = 8


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="lunarlander")
    ap.add_argument("--steps-per-launch", type=int, default=250,
                    help="collection steps per fused launch (where the workload has a fused collection kernel)")
    ap.add_argument("--update-minibatches", type=int, default=200,
                    help="minibatches of 4096 timed for the PPO-update figure")
    ap.add_argument("--preroll", type=int, default=400,
                    help="untimed collection steps before the warm-up, so that the timed steps see the steady-state "
                         "mix of flight, contacts, finished episodes and resets instead of a fresh reset's free fall")
    ap.add_argument("--min-timed-ms", type=float, default=150.0,
                    help="the timed region of `steps` steps is repeated until this much time has been measured; "
                         "the median repeat is reported")
    ap.add_argument("--full-update", action="store_true",
                    help="after the rollout, time the whole PPO update of the collected batch as the reference runs "
                         "it: bootstrap values, reward normalisation (continuous agents), GAE, advantage normalisation, "
                         "then --epochs epochs of (device permutation + every whole minibatch of 4096).  With "
                         "--workload halfcheetah --steps 1000 this is the full update of the HalfCheetah configuration: "
                         "10 epochs x 1000 minibatches on 4 096 000 samples")
    ap.add_argument("--epochs", type=int, default=10, help="epochs of --full-update")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 64 MiB read + 64 MiB write elementwise kernel 10 times, the "
                         "known-size reference for scaling FETCH_SIZE / WRITE_SIZE counter readings")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one MI355X; --gpus %d is not supported "
                 "(no collective or multi-GPU path is part of it)" % args.gpus)

    import numpy as np
    import torch
    mrl = importlib.import_module("mojo-rl_amd")
    ctx = mrl.DeviceContext("cuda:0")
    env_name, N_ENVS, HIDDEN, ACT, ENV_STEP_BYTES, describe = WORKLOADS[args.workload]
    E = getattr(mrl, env_name)
    OBS = E.OBS_DIM
    actor, critic, continuous = build_nets(mrl, E, HIDDEN, ACT)
    FWD_FLOPS = fwd_flops(E, HIDDEN)
    T = max(args.steps, 1)
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N_ENVS, T, done_cap=4 * N_ENVS + 64 * T)
    # reference initialisers: Xavier for the discrete agent, Kaiming + small Gaussian head for the
    # continuous one (deep_agents/ppo/ppo.mojo:807-817, ppo_continuous.mojo:171-342)
    init = mrl.Kaiming if continuous else mrl.Xavier
    anet = mrl.Network(ctx, actor, mrl.Adam(lr=3e-4), init(seed=0x5EED + 2))
    cnet = mrl.Network(ctx, critic, mrl.Adam(lr=1e-3), init(seed=0x5EED + 3))
    if continuous:
        mrl.init_params_small(ctx, anet.params, OBS * HIDDEN + HIDDEN + HIDDEN * HIDDEN + HIDDEN, HIDDEN,
                              E.ACTION_DIM, seed=0x5EED + 4)
    rb.actor_params, rb.critic_params = anet.params, cnet.params
    E.reset_kernel_gpu(ctx, rb.states, 0x5EED + 2)
    rb.obs.copy_(rb.states.view(N_ENVS, E.STATE_SIZE)[:, :OBS].reshape(-1))
    desc = rb.descriptor()

    fused = mrl.ppo.rollout_fused(desc)
    SPL = max(1, min(args.steps_per_launch, T)) if fused else 1   # collection steps per launch
    # untimed: the envs are taken from the reset into the steady-state episode mix, then the warm-up;
    # fused launches have the shape of the timed ones (SPL steps) as far as the counts allow, so that a
    # kernel trace of the run averages over launches of one kind
    done = 0
    for phase, count in (("preroll", args.preroll), ("warmup", min(args.warmup, T))):
        left = count
        while left > 0:
            n = min(SPL if fused else T, left)
            mrl.ppo.rollout_steps(ctx, desc, 0, n, 7 + done, 1, 0, 0, 9000 + done, 1)
            done += n
            left -= n
    ctx.synchronize()
    rb.done_count.zero_()
    ctx.synchronize()

    # ---- timed region: exactly `steps` collection steps through mrl_rollout_steps, bracketed by
    # synchronisations.  Where that is one fused launch per call, every launch is bracketed by HIP
    # events; where it issues two kernels per step, the events go around the kernels of every 8th step
    # (an event between two launches costs device time, about 3 us each here, so timing every step
    # would slow the region it measures).  A short region (the default of a driver that asks for a few
    # steps) is repeated, the envs carrying on from where they are, until min-timed-ms has been
    # measured; the line reports the median repeat.
    def timed_region(rep):
        ctx.profile_begin(4 * T + 16, sample_every=1 if fused else EVENT_STRIDE)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for c in range(0, T, SPL if fused else T):
            n = min(SPL, T - c) if fused else T
            mrl.ppo.rollout_steps(ctx, desc, c, n, 1000 + c + rep * T, 1, 0, 0, 50000 + c + rep * T, 1)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, ctx.profile_end()

    runs, spent = [], 0.0
    while True:
        dt_r, ph_r = timed_region(len(runs))
        runs.append((dt_r, ph_r))
        spent += dt_r
        if spent * 1e3 >= args.min_timed_ms or len(runs) >= 400:
            break
    runs.sort(key=lambda x: x[0])
    dt, phases = runs[len(runs) // 2]
    env_steps_per_s = N_ENVS * T / dt
    episodes = int(rb.done_count.item())

    ph_us = {k: (1e3 * v[0] / max(v[1], 1)) for k, v in phases.items()}
    traffic = measured_traffic(SPL) if args.workload == "lunarlander" else {}
    kernels = {}
    if fused:
        # one kernel does everything: its nearest roofline is the fp32 matrix-core peak (the policy
        # forward is the only throughput-bound part; the env step is a serial chain per wavefront)
        launch_us = ph_us["collect"]
        steps_per_launch = T / max(phases["collect"][1], 1)
        tflops = FWD_FLOPS * N_ENVS * steps_per_launch / (launch_us * 1e-6) / 1e12
        act_id = 1 if ACT == "relu" else 2
        name = {"lunarlander": "mrl::collect_kernel<mrl::LunarLander, %d, %d, false>" % (HIDDEN, act_id),
                "cartpole": "mrl::collect_classic_kernel<mrl::CartPoleSlot, %d, false>" % act_id,
                "pendulum": "mrl::collect_classic_kernel<mrl::PendulumSlot, %d, true>" % act_id,
                "bipedal": "mrl::collect_walker_kernel<mrl::BipedalWalker, %d, false>" % act_id,
                "halfcheetah": "mrl::collect_walker_kernel<mrl::HalfCheetah16, %d, true>" % act_id,
                "carracing": "mrl::collect_car_kernel<%d>" % act_id,
                "hopper": "mrl::collect_planar_kernel<mrl::planar::Hopper, %d>" % act_id,
                "walker2d": "mrl::collect_planar_kernel<mrl::planar::Walker2d, %d>" % act_id}[args.workload]
        roofline = {"kernel": name + " (policy forward + sampling + env step + auto-reset + rollout stores, %d steps per launch)" % steps_per_launch,
                    "bound": "mfma", "achieved": tflops, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                    "frac": tflops / MFMA_FP32_PEAK_TFLOPS,
                    # the counters were read at 250 and at 20 steps per launch: no figure for other shapes
                    "traffic": traffic.get(name) if steps_per_launch == SPL else None,
                    "avg_launch_us": launch_us, "steps_per_launch": steps_per_launch,
                    "us_per_step": launch_us / steps_per_launch}
        kernels["collect_TFLOPs"] = tflops
        # the same steps issued as two kernels per step (mrl_rollout_step), for comparison
        T2 = min(T, 200)
        ctx.profile_begin(4 * T2 + 16, sample_every=EVENT_STRIDE)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for t in range(T2):
            mrl.ppo.rollout_step(ctx, desc, t, 3000 + t, 0, 70000 + t)
        torch.cuda.synchronize()
        dt2 = time.perf_counter() - t2
        ph2 = ctx.profile_end()
        ph2_us = {k: (1e3 * v[0] / max(v[1], 1)) for k, v in ph2.items()}
        two = {"steps": T2, "env_steps_per_s": N_ENVS * T2 / dt2, "us_per_step": 1e6 * dt2 / T2,
               "policy_kernel_us": ph2_us["policy_fwd"], "env_step_kernel_us": ph2_us["env_step"]}
        fwd_us, env_us = ph2_us["policy_fwd"], ph2_us["env_step"]
    else:
        two = None
        fwd_us, env_us = ph_us["policy_fwd"], ph_us["env_step"]
    fwd_tflops = FWD_FLOPS * N_ENVS / (fwd_us * 1e-6) / 1e12
    env_gbs = ENV_STEP_BYTES * N_ENVS / (env_us * 1e-6) / 1e9
    if not fused:
        if fwd_us >= env_us:
            name = "mrl::policy_kernel<%d, %d, %s>" % (HIDDEN, 1 if ACT == "relu" else 2, "true" if continuous else "false")
            roofline = {"kernel": name + " (actor + critic forward, sampling, stores)", "bound": "mfma",
                        "achieved": fwd_tflops, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                        "frac": fwd_tflops / MFMA_FP32_PEAK_TFLOPS, "traffic": traffic.get(name),
                        "avg_launch_us": fwd_us}
        else:
            name = {"lunarlander": "mrl::phys_step_kernel<mrl::LunarLander, true>",
                    "bipedal": "mrl::phys_step_kernel<mrl::BipedalWalker, true>",
                    "halfcheetah": "mrl::hc_lanes_step_kernel<true>", "carracing": "mrl::car_step_kernel<true>",
                    "cartpole": "mrl::cartpole_step_kernel", "pendulum": "mrl::pendulum_step_kernel",
                    "hopper": "mrl::planar_step_kernel<mrl::planar::Hopper, true>",
                    "walker2d": "mrl::planar_step_kernel<mrl::planar::Walker2d, true>"}[args.workload]
            roofline = {"kernel": name + " (env step + auto-reset + post-step stores)", "bound": "hbm",
                        "achieved": env_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": env_gbs / HBM_PEAK_GBS,
                        "traffic": traffic.get(name), "avg_launch_us": env_us}

    # ---- PPO update on the collected batch (minibatch 4096, reference defaults)
    MB = min(4096, N_ENVS * T)
    cls = mrl.ppo.ContinuousUpdate if continuous else mrl.ppo.DiscreteUpdate
    upd = cls(ctx, rb, MB, anet.optimizer, cnet.optimizer, target_kl=0.0, normalize_rewards=continuous)
    upd.compute_advantages()
    total = N_ENVS * T
    n_mb = max(1, min(args.update_minibatches, total // MB))
    perm = upd.indices
    mrl.ppo.permutation(ctx, perm, 0x5EED)
    for k in range(min(3, n_mb)):
        upd.minibatch_step(perm[k * MB:(k + 1) * MB])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    upd.run_epoch(perm[:n_mb * MB])
    torch.cuda.synchronize()
    dtu = time.perf_counter() - t1
    update_sps = n_mb * MB / dtu
    t2 = time.perf_counter()
    upd.compute_advantages()
    torch.cuda.synchronize()
    gae_ms = (time.perf_counter() - t2) * 1e3

    full = None
    if args.full_update:
        # deep_agents/ppo/ppo_continuous.mojo:2852-3260 (ppo.mojo:2296-2727): phases 2 and 3 of one train_gpu
        # iteration on the batch just collected, no early stop (target_kl = 0)
        per_epoch = total // MB
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        ran = upd.update(args.epochs, seed=0x5EED)
        torch.cuda.synchronize()
        dtf = time.perf_counter() - t3
        finite = bool(torch.isfinite(anet.params).all().item() and torch.isfinite(cnet.params).all().item())
        full = {"epochs": ran, "minibatches_per_epoch": per_epoch, "minibatch": MB, "batch_samples": total,
                "samples_processed": ran * per_epoch * MB, "ms": 1e3 * dtf,
                "samples_per_s": ran * per_epoch * MB / dtf, "ms_per_minibatch": 1e3 * dtf / max(1, ran * per_epoch),
                "includes": "bootstrap value forward, reward normalisation (continuous), GAE, advantage normalisation, "
                            "per epoch one device permutation and every whole minibatch (forward, loss gradients, "
                            "backward, clip, Adam)",
                "adam_steps_taken": anet.optimizer.t, "parameters_finite": finite}

    # the env-step kernel against the HBM roofline where it does best (a batch that fills the chip many
    # times over), beside the figure at the workload's own batch in env_step_GBs / env_step_frac_hbm
    env_peak = env_step_at_large_batch(mrl, ctx, torch, E, args.workload, ENV_STEP_BYTES)

    out = {
        "metric": "env-steps/s incl. policy fwd on 1 MI355X; PPO update samples/s",
        "value": env_steps_per_s, "unit": "env-steps/s", "n_gpus": 1, "steps": T, "warmup": args.warmup,
        "ms_per_step": 1e3 * dt / T, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": describe + "; update: minibatch %d, clip 0.2, Adam" % MB,
                   "n_envs": N_ENVS, "rollout_steps": T, "minibatch": MB},
        "ppo_update_samples_per_s": update_sps,
        "ppo_update": {"minibatches_timed": n_mb, "ms_per_minibatch": 1e3 * dtu / n_mb,
                       "gae_plus_normalise_ms": gae_ms},
        "timed_repeats": len(runs), "timed_ms_total": 1e3 * spent, "preroll_steps": args.preroll,
        "episodes_finished": episodes,
        "phase_us": ph_us,
        "phase_events": ({"launches_timed": phases["collect"][1], "steps_per_launch": SPL} if fused else
                         {"sampled_every_n_steps": EVENT_STRIDE, "launches_timed": phases["env_step"][1]}),
        "kernels": dict(kernels, policy_fwd_TFLOPs=fwd_tflops, env_step_GBs=env_gbs,
                        env_step_frac_hbm=env_gbs / HBM_PEAK_GBS,
                        policy_fwd_frac_mfma=fwd_tflops / MFMA_FP32_PEAK_TFLOPS,
                        update_TFLOPs=3.0 * FWD_FLOPS * update_sps / 1e12,
                        env_step_alone_at_large_batch=env_peak),
        "roofline": roofline,
    }
    if full is not None:
        out["full_update_samples_per_s"] = full["samples_per_s"]
        out["full_update"] = full
    if two is not None:
        out["two_kernels_per_step"] = two
    if args.copy_calibration:
        src = torch.ones(16 * 1024 * 1024, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(10):
            torch.add(src, 1.0, out=dst)
        torch.cuda.synchronize()
        out["copy_calibration"] = {"kernel": "at::native::vectorized_elementwise_kernel (add scalar)",
                                   "bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4, "launches": 10}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(np)
    ctx.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
