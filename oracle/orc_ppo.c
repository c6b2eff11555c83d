/*
 * PPO utilities: CPU restatement (test infrastructure, never shipped).
 *
 *   categorical sampler   deep_agents/ppo/ppo.mojo:4064-4123
 *   gaussian sampler      deep_agents/ppo/kernels.mojo:12-98
 *   GAE                   deep_agents/ppo/ppo.mojo:2317-2353 (time-major, idx = t*N + env)
 *   advantage norm        ppo.mojo:2356-2371 (rollout-wide, serial fp32 sums),
 *                         ppo.mojo:2478-2511 + :637-653 (per minibatch, host stats),
 *                         kernels.mojo:507-599 (per minibatch, single block)
 *   actor grad discrete   ppo.mojo:285-378
 *   actor grad gaussian   kernels.mojo:230-412
 *   critic grad           ppo.mojo:538-633 (convention 0), kernels.mojo:416-486 (convention 1)
 *   grad-norm clip        ppo.mojo:382-534 / kernels.mojo:740-805
 *   Adam                  deep_rl/optimizer/adam.mojo:52-105
 *   log_std clamp         kernels.mojo:842-873
 *   RunningMeanStd        core/utils/normalization.mojo:188-292
 *
 * The loss-gradient formulas exist in the reference only as per-sample GPU kernels;
 * they are restated here as the scalar functions they are.  Sums that the reference
 * performs as LDS tree reductions are taken serially in fp32 here; tests compare
 * them with a tolerance, not bit-for-bit.
 */
#include <math.h>
#include "orc.h"

/* fp32 exp / log / cos as the correctly rounded value (through the Float64 routine, rounded once):
 * the sampled action index, the PPO ratio and its clip test depend on the last bit, and the
 * correctly rounded value is the one result that two independent math libraries agree on */
static inline float f32_exp(float x) { return (float)exp((double)x); }
static inline float f32_log(float x) { return (float)log((double)x); }
static inline float f32_cos(float x) { return (float)cos((double)x); }

void orc_sample_categorical(const float *logits, int n, int A, uint32_t seed, float *actions,
                            float *log_probs) {
    for (int i = 0; i < n; ++i) {
        const float *l = logits + (long)i * A;
        uint32_t rng = seed ^ ((uint32_t)i * 2654435761u);
        rng = orc_xorshift32(rng);
        float max_logit = l[0];
        for (int a = 1; a < A; ++a) if (l[a] > max_logit) max_logit = l[a];
        float sum_exp = 0.0f;
        for (int a = 0; a < A; ++a) sum_exp = sum_exp + f32_exp(l[a] - max_logit);
        float u = orc_random_uniform(&rng);
        float cumsum = 0.0f;
        int sel = 0;
        for (int a = 0; a < A; ++a) {
            float prob = f32_exp(l[a] - max_logit) / sum_exp;
            cumsum = cumsum + prob;
            if (u < cumsum) { sel = a; break; }
        }
        actions[i] = (float)sel;
        float p = f32_exp(l[sel] - max_logit) / sum_exp;
        log_probs[i] = f32_log(p + 1e-8f);
    }
}

void orc_sample_gaussian(const float *actor_out, int n, int A, uint64_t seed, float *actions,
                         float *log_probs) {
    const float EPS = 1e-6f, LOG_2PI = (float)1.8378770664093453;
    for (int i = 0; i < n; ++i) {
        float total = 0.0f;
        for (int j = 0; j < A; ++j) {
            float mean = actor_out[(long)i * 2 * A + j];
            float log_std = actor_out[(long)i * 2 * A + A + j];
            if (log_std < -5.0f) log_std = -5.0f;
            else if (log_std > 2.0f) log_std = 2.0f;
            float rv[4];
            orc_philox_uniform4((uint64_t)((int64_t)seed + (int64_t)i * A + j), 0, 0, rv);
            float u1 = rv[0] + 1e-8f;
            float mag = sqrtf(-2.0f * f32_log(u1));
            float noise = mag * f32_cos(rv[1] * (float)6.283185307179586);
            float std = f32_exp(log_std);
            float action = mean + std * noise;
            actions[(long)i * A + j] = action;
            float an = (action - mean) / (std + EPS);
            float lg = -0.5f * (LOG_2PI + 2.0f * log_std + an * an);
            total = total + lg;
        }
        log_probs[i] = total;
    }
}

/* add_obs_noise_kernel, deep_agents/ppo/kernels.mojo:882-925 */
void orc_add_obs_noise(float *obs, int n, int obs_dim, float noise_std, uint32_t seed) {
    if (!(noise_std > 0.0f)) return;
    for (int i = 0; i < n; ++i) {
        for (int d = 0; d < obs_dim; ++d) {
            float rv[4];
            orc_philox_uniform4((uint64_t)((int64_t)seed + (int64_t)i * obs_dim + d), 0, 0, rv);
            float u1_safe = rv[0] + 1e-8f;
            float mag = sqrtf(-2.0f * f32_log(u1_safe));
            float noise = mag * f32_cos(rv[1] * (float)6.283185307179586);
            obs[(long)i * obs_dim + d] = obs[(long)i * obs_dim + d] + noise * noise_std;
        }
    }
}

void orc_gae(int T, int N, const float *rewards, const float *values, const float *dones,
             const float *bootstrap, double gamma, double lam, float *adv, float *ret) {
    const float g = (float)gamma;
    const float decay = (float)(gamma * lam);
    for (int e = 0; e < N; ++e) {
        float gae = 0.0f;
        for (int t = T - 1; t >= 0; --t) {
            long idx = (long)t * N + e;
            float next_val = (t == T - 1) ? bootstrap[e] : values[idx + N];
            if (dones[idx] > 0.5f) { next_val = 0.0f; gae = 0.0f; }
            float delta = rewards[idx] + g * next_val - values[idx];
            gae = delta + decay * gae;
            adv[idx] = gae;
            ret[idx] = gae + values[idx];
        }
    }
}

void orc_normalize_advantages(float *a, int n) {
    float mean = 0.0f, var_sum = 0.0f;
    for (int i = 0; i < n; ++i) mean += a[i];
    mean /= (float)n;
    for (int i = 0; i < n; ++i) { float d = a[i] - mean; var_sum += d * d; }
    float variance = var_sum / (float)n;
    float std = sqrtf(variance + 1e-8f);
    for (int i = 0; i < n; ++i) a[i] = (a[i] - mean) / (std + 1e-8f);
}

void orc_normalize_minibatch_host(float *a, int n) {
    float mean = 0.0f, var_sum = 0.0f;
    for (int i = 0; i < n; ++i) mean += a[i];
    mean /= (float)n;
    for (int i = 0; i < n; ++i) { float d = a[i] - mean; var_sum += d * d; }
    float std = sqrtf(var_sum / (float)n + 1e-8f);
    for (int i = 0; i < n; ++i) a[i] = (a[i] - mean) / (std + 1e-8f);
}

void orc_normalize_minibatch_fused(float *a, int n) {
    float sum = 0.0f, var_sum = 0.0f;
    for (int i = 0; i < n; ++i) sum += a[i];
    float mean = sum / (float)n;
    for (int i = 0; i < n; ++i) { float d = a[i] - mean; var_sum += d * d; }
    float variance = var_sum / (float)n;
    /* sqrt(variance + 1e-8) with a Float64 literal promotes through fp32 in the kernel */
    float std = sqrtf(variance + 1e-8f);
    for (int i = 0; i < n; ++i) a[i] = (a[i] - mean) / (std + 1e-8f);
}

void orc_ppo_actor_grad_discrete(const float *logits, const float *old_logp, const float *adv,
                                 const float *actions, int mb, int A, float clip_eps,
                                 float ent_coef, float *grad_logits, float *kl) {
    for (int b = 0; b < mb; ++b) {
        const float *l = logits + (long)b * A;
        int action = (int)actions[b];
        float advantage = adv[b];
        float max_logit = l[0];
        for (int a = 1; a < A; ++a) if (l[a] > max_logit) max_logit = l[a];
        float sum_exp = 0.0f;
        for (int a = 0; a < A; ++a) sum_exp = sum_exp + f32_exp(l[a] - max_logit);
        float probs[64];
        for (int a = 0; a < A; ++a) probs[a] = f32_exp(l[a] - max_logit) / sum_exp;
        float new_logp = f32_log(probs[action] + 1e-8f);
        kl[b] = old_logp[b] - new_logp;
        float ratio = f32_exp(new_logp - old_logp[b]);
        int clipped = (ratio < 1.0f - clip_eps) || (ratio > 1.0f + clip_eps);
        for (int a = 0; a < A; ++a) {
            if (clipped) { grad_logits[(long)b * A + a] = 0.0f; continue; }
            float d_log_prob = (a == action) ? 1.0f - probs[a] : -probs[a];
            float log_prob_ent = f32_log(probs[a] + 1e-8f);
            float d_entropy = -probs[a] * (1.0f + log_prob_ent);
            grad_logits[(long)b * A + a] =
                (-advantage * ratio * d_log_prob - ent_coef * d_entropy) / (float)mb;
        }
    }
}

void orc_ppo_actor_grad_gaussian(const float *actor_out, const float *old_logp, const float *adv,
                                 const float *actions, int mb, int A, float clip_eps,
                                 float ent_coef, float *grad_out, float *kl_out) {
    const float eps = 1e-6f, log_2pi = (float)1.8378770664093453;
    for (int b = 0; b < mb; ++b) {
        float advantage = adv[b], old_log_prob = old_logp[b];
        float new_log_prob = 0.0f;
        float av[32], mv[32], sv[32];
        for (int j = 0; j < A; ++j) {
            float mean = actor_out[(long)b * 2 * A + j];
            float log_std = actor_out[(long)b * 2 * A + A + j];
            float action = actions[(long)b * A + j];
            if (log_std < -5.0f) log_std = -5.0f;
            else if (log_std > 2.0f) log_std = 2.0f;
            float std = f32_exp(log_std);
            float an = (action - mean) / (std + eps);
            av[j] = action; mv[j] = mean; sv[j] = std;
            float lg = -0.5f * (log_2pi + 2.0f * log_std + an * an);
            new_log_prob = new_log_prob + lg;
        }
        float diff = new_log_prob - old_log_prob;
        if (diff > 20.0f) diff = 20.0f;
        else if (diff < -20.0f) diff = -20.0f;
        float ratio = f32_exp(diff);
        float kl = (ratio - 1.0f) - diff;
        if (kl < 0.0f) kl = 0.0f;
        else if (kl > 100.0f) kl = 100.0f;
        kl_out[b] = kl;
        float clipped_ratio = ratio;
        if (clipped_ratio < 1.0f - clip_eps) clipped_ratio = 1.0f - clip_eps;
        else if (clipped_ratio > 1.0f + clip_eps) clipped_ratio = 1.0f + clip_eps;
        float unclipped_obj = ratio * advantage;
        float clipped_obj = clipped_ratio * advantage;
        int is_clipped = clipped_obj < unclipped_obj;
        for (int j = 0; j < A; ++j) {
            float *gm = grad_out + (long)b * 2 * A + j;
            float *gs = grad_out + (long)b * 2 * A + A + j;
            if (is_clipped) { *gm = 0.0f; *gs = 0.0f; continue; }
            float an = (av[j] - mv[j]) / (sv[j] + eps);
            float d_mean = an / (sv[j] + eps);
            float d_log_std = an * an - 1.0f;
            float grad_mean = (-advantage * ratio * d_mean) / (float)mb;
            float grad_log_std = (-advantage * ratio * d_log_std - ent_coef * 1.0f) / (float)mb;
            if (grad_mean > 10.0f) grad_mean = 10.0f;
            else if (grad_mean < -10.0f) grad_mean = -10.0f;
            if (grad_log_std > 10.0f) grad_log_std = 10.0f;
            else if (grad_log_std < -10.0f) grad_log_std = -10.0f;
            *gm = grad_mean; *gs = grad_log_std;
        }
    }
}

void orc_ppo_critic_grad(const float *values, const float *old_values, const float *returns, int mb,
                         int convention, int clipped, float value_coef, float clip_eps, float *grad) {
    for (int b = 0; b < mb; ++b) {
        float v = values[b], ret = returns[b];
        if (convention == 0) {
            if (!clipped) {
                grad[b] = 2.0f * value_coef * (v - ret) / (float)mb;
                continue;
            }
            float v_old = old_values[b];
            float v_diff = v - v_old;
            float v_clipped;
            if (v_diff > clip_eps) v_clipped = v_old + clip_eps;
            else if (v_diff < -clip_eps) v_clipped = v_old - clip_eps;
            else v_clipped = v;
            float loss_unclipped = (v - ret) * (v - ret);
            float loss_clipped = (v_clipped - ret) * (v_clipped - ret);
            float g;
            if (loss_unclipped > loss_clipped) g = 2.0f * (v - ret);
            else if (v_diff > clip_eps || v_diff < -clip_eps) g = 0.0f;
            else g = 2.0f * (v - ret);
            grad[b] = value_coef * g / (float)mb;
        } else {
            if (!clipped) {
                grad[b] = (v - ret) / (float)mb;
                continue;
            }
            float old_value = old_values[b];
            float d = v - old_value;
            float mn = d < clip_eps ? d : clip_eps;        /* min(value - old, eps) */
            float mx = mn > -clip_eps ? mn : -clip_eps;    /* max(.., -eps) */
            float value_clipped = old_value + mx;
            float loss_unclipped = (v - ret) * (v - ret);
            float loss_clipped = (value_clipped - ret) * (value_clipped - ret);
            if (loss_clipped > loss_unclipped) {
                float clip_sign = 1.0f;
                if (v - old_value > clip_eps) clip_sign = 0.0f;
                else if (v - old_value < -clip_eps) clip_sign = 0.0f;
                grad[b] = clip_sign * (value_clipped - ret) / (float)mb;
            } else {
                grad[b] = (v - ret) / (float)mb;
            }
        }
    }
}

float orc_clip_grad_norm(float *g, int n, float max_norm) {
    float total = 0.0f;
    for (int i = 0; i < n; ++i) total += g[i] * g[i];
    float norm = sqrtf(total);
    float scale = 1.0f;
    if (norm > max_norm) scale = max_norm / (norm + 1e-8f);
    for (int i = 0; i < n; ++i) g[i] = g[i] * scale;
    return scale;
}

void orc_adam_step(float *p, const float *g, float *state, int n, int t, double lr, double b1,
                   double b2, double eps) {
    float bc1 = (float)(1.0 - pow(b1, (double)t));
    float bc2 = (float)(1.0 - pow(b2, (double)t));
    float omb1 = (float)(1.0 - b1), omb2 = (float)(1.0 - b2);
    float beta1 = (float)b1, beta2 = (float)b2, lrf = (float)lr, epsf = (float)eps;
    for (int i = 0; i < n; ++i) {
        float gi = g[i], m = state[2 * i], v = state[2 * i + 1];
        float m_new = beta1 * m + omb1 * gi;
        float v_new = beta2 * v + omb2 * gi * gi;
        state[2 * i] = m_new; state[2 * i + 1] = v_new;
        float m_hat = m_new / bc1, v_hat = v_new / bc2;
        p[i] -= lrf * m_hat / (sqrtf(v_hat) + epsf);
    }
}

void orc_clamp_log_std(float *params, int offset, int A) {
    for (int i = 0; i < A; ++i) {
        float v = params[offset + i];
        if (v < -5.0f) params[offset + i] = -5.0f;
        else if (v > 2.0f) params[offset + i] = 2.0f;
    }
}

void orc_rms_update(orc_rms *r, const float *x, int n) {
    if (n == 0) return;
    double bm = 0.0;
    for (int i = 0; i < n; ++i) bm += (double)x[i];
    bm /= (double)n;
    double bv = 0.0;
    for (int i = 0; i < n; ++i) { double d = (double)x[i] - bm; bv += d * d; }
    bv /= (double)n;
    double new_count = r->count + (double)n;
    if (r->count == 0) {
        r->mean = bm;
        r->var_sum = bv * (double)n;
    } else {
        double delta = bm - r->mean;
        double new_mean = r->mean + delta * (double)n / new_count;
        r->var_sum = r->var_sum + bv * (double)n + delta * delta * r->count * (double)n / new_count;
        r->mean = new_mean;
    }
    r->count = new_count;
}

void orc_rms_normalize(const orc_rms *r, float *x, int n) {
    double var = (r->count < 2) ? 1.0 : r->var_sum / r->count;
    double std = sqrt(var + 1e-8);
    for (int i = 0; i < n; ++i) x[i] = (float)(((double)x[i] - r->mean) / (std + 1e-8));
}

/* Fisher-Yates shuffle of the indices 0 .. n-1 on supplied uniforms (core/utils/shuffle.mojo:21-48;
 * the same loop inline in deep_agents/ppo/ppo.mojo:2425-2434): for i = n-1 down to 1,
 * j = Int(u * Float64(i + 1)) with u the next draw of random_float64() -- here u[n-1-i], the draws in
 * the order the loop consumes them -- clamped to i (shuffle.mojo:42-43; a draw in [0, 1) never needs
 * it), then indices[i] <-> indices[j]. */
void orc_shuffle_indices(int n, const double *u, int32_t *indices) {
    for (int i = 0; i < n; ++i) indices[i] = i;
    for (int i = n - 1; i > 0; --i) {
        int j = (int)(u[n - 1 - i] * (double)(i + 1));
        if (j > i) j = i;
        const int32_t tmp = indices[i];
        indices[i] = indices[j];
        indices[j] = tmp;
    }
}
