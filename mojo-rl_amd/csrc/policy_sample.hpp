// Action sampling of one env from its policy head, shared by the fused policy kernel, the fused
// collection kernel and the stand-alone sampling kernels.
#pragma once
#include "mrl_device.hpp"

namespace mrl {

// Categorical sampling from A logits (deep_agents/ppo/ppo.mojo:4064-4123): xorshift32 stream
// keyed by (seed, env index), inverse-CDF draw, log-probability of the drawn action.
MRL_DEV void sample_categorical(const float *l, int A, uint32_t seed, int i, int &sel, float &logp) {
    uint32_t rng = seed ^ ((uint32_t)i * 2654435761u);
    rng = xorshift32(rng);
    float max_logit = l[0];
    for (int a = 1; a < A; ++a) if (l[a] > max_logit) max_logit = l[a];
    float sum_exp = 0.0f;
    for (int a = 0; a < A; ++a) sum_exp = sum_exp + exp32(l[a] - max_logit);
    const float u = random_uniform(rng);
    float cumsum = 0.0f;
    sel = 0;
    for (int a = 0; a < A; ++a) {
        float prob = exp32(l[a] - max_logit) / sum_exp;
        cumsum = cumsum + prob;
        if (u < cumsum) { sel = a; break; }
    }
    const float pr = exp32(l[sel] - max_logit) / sum_exp;
    logp = log32(pr + 1e-8f);
}

// The same draw for at most SAMPLE_A_MAX actions (the fused kernels' policy heads), bit for bit.
constexpr int SAMPLE_A_MAX = 8;
MRL_DEV void sample_categorical_few(const float *l, int A, uint32_t seed, int i, int &sel, float &logp) {
    uint32_t rng = seed ^ ((uint32_t)i * 2654435761u);
    rng = xorshift32(rng);
    float max_logit = l[0];
    for (int a = 1; a < A; ++a) if (l[a] > max_logit) max_logit = l[a];
    // every exponential is taken once and kept (the reference recomputes them for the probabilities and for
    // the drawn action: the same values); all slots are walked so that the array stays in registers
    float e[SAMPLE_A_MAX];
    float sum_exp = 0.0f;
#pragma unroll
    for (int a = 0; a < SAMPLE_A_MAX; ++a) {
        e[a] = 0.0f;
        if (a < A) {
            e[a] = exp32(l[a] - max_logit);
            sum_exp = sum_exp + e[a];
        }
    }
    const float u = random_uniform(rng);
    float cumsum = 0.0f, e_sel = e[0];
    bool found = false;
    sel = 0;
#pragma unroll
    for (int a = 0; a < SAMPLE_A_MAX; ++a) {
        if (a < A) {
            const float prob = e[a] / sum_exp;
            cumsum = cumsum + prob;
            if (!found && u < cumsum) {
                sel = a;
                e_sel = e[a];
                found = true;
            }
        }
    }
    const float pr = e_sel / sum_exp;
    logp = log32(pr + 1e-8f);
}

// Gaussian sampling (deep_agents/ppo/kernels.mojo:12-98) of components j0 .. j0 + m of an action
// with A components: one Philox stream per (env, component), Box-Muller, clamped log_std;
// returns the summed log-probability of those components and leaves them in act[0 .. m).
// std_p (optional): exp of the clamped log_std of the same components, taken ahead by a caller whose
// log_std does not change from call to call.
MRL_DEV float gaussian_log_std(float log_std) { return log_std < -5.0f ? -5.0f : (log_std > 2.0f ? 2.0f : log_std); }
MRL_DEV float sample_gaussian_part(const float *mean, const float *log_std_p, int m, int A, int j0,
                                   uint32_t seed, int i, float *act, const float *std_p = nullptr) {
    const float EPS = 1e-6f, LOG_2PI = (float)1.8378770664093453;
    float total = 0.0f;
    for (int j = 0; j < m; ++j) {
        const float mu = mean[j];
        const float log_std = gaussian_log_std(log_std_p[j]);
        Uniform4 rv = philox_uniform4((uint64_t)((int64_t)seed + (int64_t)i * A + j0 + j), 0, 0);
        const float u1 = rv.v[0] + 1e-8f;
        const float mag = sqrtf(-2.0f * log32(u1));
        const float noise = mag * cos32(rv.v[1] * (float)6.283185307179586);
        const float std = std_p != nullptr ? std_p[j] : exp32(log_std);
        const float action = mu + std * noise;
        act[j] = action;
        const float an = (action - mu) / (std + EPS);
        total = total + -0.5f * (LOG_2PI + 2.0f * log_std + an * an);
    }
    return total;
}
MRL_DEV float sample_gaussian(const float *mean_row, const float *log_std_p, int A, uint32_t seed, int i,
                              float *act, const float *std_p = nullptr) {
    return sample_gaussian_part(mean_row, log_std_p, A, A, 0, seed, i, act, std_p);
}

}  // namespace mrl
