// Arguments of the fused collection kernels (many rollout steps of a block's envs in one launch) and
// the entry of the walkers' kernel, which lives in a translation unit of its own.
#pragma once
#include "mrl_host.hpp"

namespace mrl {

struct CollectArgs {
    float *states, *obs;                  // [N][STATE], [N][OBS]
    const float *actor_p, *critic_p, *shapes;
    int n_envs, A, t0, n_steps;
    uint32_t sample_seed, sample_stride;
    uint64_t reset_seed, reset_stride;
    float *r_obs, *r_actions, *r_logp, *r_values, *r_rewards, *r_dones;   // time-major, row 0
    Accounting acc;                       // r_rewards / r_dones unused here (set per step)
    unsigned spin_limit;                  // polls before a wait at a wavefront-group barrier gives up
    int *sync_error;                      // raised (host-visible) by a workgroup whose wait gave up
    int car_trait_form;                   // CarRacingV2: reward / termination arithmetic of the GPU trait's step
};

// BipedalWalker / HalfCheetah with the agents' 256-wide Gaussian nets: true when `a` was launched
bool collect_walker_fusable(const mrl_rollout *r, int *act);
int launch_collect_walker(mrl_ctx *ctx, const mrl_rollout *r, const CollectArgs &a, int act);

}  // namespace mrl
