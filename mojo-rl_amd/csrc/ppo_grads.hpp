// Per-sample loss gradients of the PPO agents, shared by the stand-alone kernels (mrl_ppo.hip) and
// the merged kernel of the minibatch update (mrl_update.hip).
#pragma once
#include "mrl_device.hpp"

namespace mrl {

// deep_agents/ppo/ppo.mojo:285-378 for one sample: l = its A logits, g = its A gradient slots;
// returns the sample's KL estimate (old - new log-prob)
MRL_DEV float actor_grad_discrete_row(const float *l, int action, float advantage, float old, int mb, int A,
                                      float clip_eps, float ent_coef, float *g_row) {
    float max_logit = l[0];
    for (int a = 1; a < A; ++a) if (l[a] > max_logit) max_logit = l[a];
    // every exponential once (the reference takes exp(l[a] - max) again for the probabilities and for the
    // gradient: the same values); heads wider than the array fall back to recomputing
    constexpr int KEEP = 8;
    float e[KEEP];
    float sum_exp = 0.0f;
#pragma unroll
    for (int a = 0; a < KEEP; ++a) {
        e[a] = 0.0f;
        if (a < A) {
            e[a] = exp32(l[a] - max_logit);
            sum_exp = sum_exp + e[a];
        }
    }
    for (int a = KEEP; a < A; ++a) sum_exp = sum_exp + exp32(l[a] - max_logit);
    float p_action = 0.0f;
#pragma unroll
    for (int a = 0; a < KEEP; ++a)
        if (a < A && a == action) p_action = e[a] / sum_exp;
    for (int a = KEEP; a < A; ++a)
        if (a == action) p_action = exp32(l[a] - max_logit) / sum_exp;
    float new_logp = log32(p_action + 1e-8f);
    float ratio = exp32(new_logp - old);
    bool clipped = (ratio < 1.0f - clip_eps) || (ratio > 1.0f + clip_eps);
#pragma unroll
    for (int a = 0; a < KEEP; ++a) {
        if (a < A) {
            float g = 0.0f;
            if (!clipped) {
                float p = e[a] / sum_exp;
                float d_log_prob = (a == action) ? 1.0f - p : -p;
                float log_prob_ent = log32(p + 1e-8f);
                float d_entropy = -p * (1.0f + log_prob_ent);
                g = (-advantage * ratio * d_log_prob - ent_coef * d_entropy) / (float)mb;
            }
            g_row[a] = g;
        }
    }
    for (int a = KEEP; a < A; ++a) {
        float g = 0.0f;
        if (!clipped) {
            float p = exp32(l[a] - max_logit) / sum_exp;
            float d_log_prob = (a == action) ? 1.0f - p : -p;
            float log_prob_ent = log32(p + 1e-8f);
            float d_entropy = -p * (1.0f + log_prob_ent);
            g = (-advantage * ratio * d_log_prob - ent_coef * d_entropy) / (float)mb;
        }
        g_row[a] = g;
    }
    return old - new_logp;
}
// actor_grad_discrete_row by eight lanes of a wavefront (lanes base .. base + 7, A <= 8), lane j on logit j:
// every lane takes one exponential and one entropy logarithm instead of A of each; the sums run over the
// lanes' values in the order the one-lane form adds them, so the bits are the same.  lj = logit j (anything
// for j >= A); g_out = gradient slot j (0 for j >= A); every lane returns the sample's KL estimate.
MRL_DEV float actor_grad_discrete_lanes(float lj, int j, int base, int action, float advantage, float old, int mb,
                                        int A, float clip_eps, float ent_coef, float &g_out) {
    float max_logit = __shfl(lj, base, 64);
#pragma unroll
    for (int a = 1; a < 8; ++a) {
        const float la = __shfl(lj, base + a, 64);
        if (a < A && la > max_logit) max_logit = la;
    }
    const float e = j < A ? exp32(lj - max_logit) : 0.0f;
    float sum_exp = 0.0f, e_action = 0.0f;
#pragma unroll
    for (int a = 0; a < 8; ++a) {
        const float ea = __shfl(e, base + a, 64);
        if (a < A) sum_exp = sum_exp + ea;
        if (a < A && a == action) e_action = ea;
    }
    const float p_action = (action >= 0 && action < A) ? e_action / sum_exp : 0.0f;
    const float new_logp = log32(p_action + 1e-8f);
    const float ratio = exp32(new_logp - old);
    const bool clipped = (ratio < 1.0f - clip_eps) || (ratio > 1.0f + clip_eps);
    float g = 0.0f;
    if (!clipped && j < A) {
        float p = e / sum_exp;
        float d_log_prob = (j == action) ? 1.0f - p : -p;
        float log_prob_ent = log32(p + 1e-8f);
        float d_entropy = -p * (1.0f + log_prob_ent);
        g = (-advantage * ratio * d_log_prob - ent_coef * d_entropy) / (float)mb;
    }
    g_out = g;
    return old - new_logp;
}
MRL_DEV float actor_grad_discrete_one(int b, const float *__restrict__ logits, const float *__restrict__ old_logp,
                                      const float *__restrict__ adv, const float *__restrict__ actions, int mb,
                                      int A, float clip_eps, float ent_coef, float *__restrict__ grad_logits) {
    return actor_grad_discrete_row(logits + (long)b * A, (int)actions[b], adv[b], old_logp[b], mb, A, clip_eps,
                                   ent_coef, grad_logits + (long)b * A);
}

// deep_agents/ppo/kernels.mojo:230-412 for one sample: o = [mean (A) | log_std (A)], act = its A
// action components, g = its 2A gradient slots; returns the sample's KL estimate
// ((ratio - 1) - diff, clamped)
MRL_DEV float actor_grad_gaussian_row(const float *o, const float *act, float advantage, float old_log_prob,
                                      int mb, int A, float clip_eps, float ent_coef, float *g) {
    const float eps = 1e-6f, log_2pi = (float)1.8378770664093453;
    // exp(log_std) of the first KEEP components is taken once (the reference takes it again for the
    // gradient: the same value); wider actions recompute the rest
    constexpr int KEEP = 8;
    float stdv[KEEP];
    float new_log_prob = 0.0f;
    auto clamped = [](float log_std) { return log_std < -5.0f ? -5.0f : (log_std > 2.0f ? 2.0f : log_std); };
#pragma unroll
    for (int j = 0; j < KEEP; ++j) {
        stdv[j] = 1.0f;
        if (j < A) {
            const float log_std = clamped(o[A + j]);
            stdv[j] = exp32(log_std);
            float an = (act[j] - o[j]) / (stdv[j] + eps);
            float lg = -0.5f * (log_2pi + 2.0f * log_std + an * an);
            new_log_prob = new_log_prob + lg;
        }
    }
    for (int j = KEEP; j < A; ++j) {
        const float log_std = clamped(o[A + j]);
        float std = exp32(log_std);
        float an = (act[j] - o[j]) / (std + eps);
        float lg = -0.5f * (log_2pi + 2.0f * log_std + an * an);
        new_log_prob = new_log_prob + lg;
    }
    float diff = new_log_prob - old_log_prob;
    if (diff > 20.0f) diff = 20.0f;
    else if (diff < -20.0f) diff = -20.0f;
    float ratio = exp32(diff);
    float kl = (ratio - 1.0f) - diff;
    if (kl < 0.0f) kl = 0.0f;
    else if (kl > 100.0f) kl = 100.0f;
    float clipped_ratio = ratio;
    if (clipped_ratio < 1.0f - clip_eps) clipped_ratio = 1.0f - clip_eps;
    else if (clipped_ratio > 1.0f + clip_eps) clipped_ratio = 1.0f + clip_eps;
    bool is_clipped = clipped_ratio * advantage < ratio * advantage;
    auto grads = [&](int j, float std) {
        float gm = 0.0f, gs = 0.0f;
        if (!is_clipped) {
            float an = (act[j] - o[j]) / (std + eps);
            float d_mean = an / (std + eps);
            float d_log_std = an * an - 1.0f;
            gm = (-advantage * ratio * d_mean) / (float)mb;
            gs = (-advantage * ratio * d_log_std - ent_coef * 1.0f) / (float)mb;
            if (gm > 10.0f) gm = 10.0f;
            else if (gm < -10.0f) gm = -10.0f;
            if (gs > 10.0f) gs = 10.0f;
            else if (gs < -10.0f) gs = -10.0f;
        }
        g[j] = gm;
        g[A + j] = gs;
    };
#pragma unroll
    for (int j = 0; j < KEEP; ++j)
        if (j < A) grads(j, stdv[j]);
    for (int j = KEEP; j < A; ++j) grads(j, is_clipped ? 1.0f : exp32(clamped(o[A + j])));
    return kl;
}
MRL_DEV float actor_grad_gaussian_one(int b, const float *__restrict__ actor_out, const float *__restrict__ old_logp,
                                      const float *__restrict__ adv, const float *__restrict__ actions, int mb,
                                      int A, float clip_eps, float ent_coef, float *__restrict__ grad_out) {
    return actor_grad_gaussian_row(actor_out + (long)b * 2 * A, actions + (long)b * A, adv[b], old_logp[b], mb, A,
                                   clip_eps, ent_coef, grad_out + (long)b * 2 * A);
}

// actor_grad_gaussian_row by eight lanes of a wavefront (lanes base .. base + 7, A <= 8), lane j on action
// component j (its mean, raw log_std and action; anything for j >= A): one exp(log_std) per lane, the
// log-probability summed over the lanes' terms in component order.  gm / gs = gradient slots j and A + j.
MRL_DEV float actor_grad_gaussian_lanes(float mean_j, float log_std_j, float act_j, int j, int base, float advantage,
                                        float old_log_prob, int mb, int A, float clip_eps, float ent_coef, float &gm,
                                        float &gs) {
    const float eps = 1e-6f, log_2pi = (float)1.8378770664093453;
    const float log_std = log_std_j < -5.0f ? -5.0f : (log_std_j > 2.0f ? 2.0f : log_std_j);
    const float std = j < A ? exp32(log_std) : 1.0f;
    float lg;
    {
        float an = (act_j - mean_j) / (std + eps);
        lg = -0.5f * (log_2pi + 2.0f * log_std + an * an);
    }
    float new_log_prob = 0.0f;
#pragma unroll
    for (int a = 0; a < 8; ++a) {
        const float v = __shfl(lg, base + a, 64);
        if (a < A) new_log_prob = new_log_prob + v;
    }
    float diff = new_log_prob - old_log_prob;
    if (diff > 20.0f) diff = 20.0f;
    else if (diff < -20.0f) diff = -20.0f;
    float ratio = exp32(diff);
    float kl = (ratio - 1.0f) - diff;
    if (kl < 0.0f) kl = 0.0f;
    else if (kl > 100.0f) kl = 100.0f;
    float clipped_ratio = ratio;
    if (clipped_ratio < 1.0f - clip_eps) clipped_ratio = 1.0f - clip_eps;
    else if (clipped_ratio > 1.0f + clip_eps) clipped_ratio = 1.0f + clip_eps;
    const bool is_clipped = clipped_ratio * advantage < ratio * advantage;
    gm = 0.0f; gs = 0.0f;
    if (!is_clipped && j < A) {
        float an = (act_j - mean_j) / (std + eps);
        float d_mean = an / (std + eps);
        float d_log_std = an * an - 1.0f;
        gm = (-advantage * ratio * d_mean) / (float)mb;
        gs = (-advantage * ratio * d_log_std - ent_coef * 1.0f) / (float)mb;
        if (gm > 10.0f) gm = 10.0f;
        else if (gm < -10.0f) gm = -10.0f;
        if (gs > 10.0f) gs = 10.0f;
        else if (gs < -10.0f) gs = -10.0f;
    }
    return kl;
}

// ppo.mojo:538-633 (convention 0) and kernels.mojo:416-486 (convention 1)
MRL_DEV float critic_grad_value(float v, float v_old, float ret, int mb, int convention, int clipped,
                                float value_coef, float clip_eps) {
    float out;
    if (convention == 0) {
        if (!clipped) {
            out = 2.0f * value_coef * (v - ret) / (float)mb;
        } else {
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
            out = value_coef * g / (float)mb;
        }
    } else {
        if (!clipped) {
            out = (v - ret) / (float)mb;
        } else {
            float old_value = v_old;
            float d = v - old_value;
            float mn = d < clip_eps ? d : clip_eps;
            float mx = mn > -clip_eps ? mn : -clip_eps;
            float value_clipped = old_value + mx;
            float loss_unclipped = (v - ret) * (v - ret);
            float loss_clipped = (value_clipped - ret) * (value_clipped - ret);
            if (loss_clipped > loss_unclipped) {
                float clip_sign = 1.0f;
                if (v - old_value > clip_eps) clip_sign = 0.0f;
                else if (v - old_value < -clip_eps) clip_sign = 0.0f;
                out = clip_sign * (value_clipped - ret) / (float)mb;
            } else {
                out = (v - ret) / (float)mb;
            }
        }
    }
    return out;
}

MRL_DEV float critic_grad_one(int b, const float *__restrict__ values, const float *__restrict__ old_values,
                              const float *__restrict__ returns, int mb, int convention, int clipped,
                              float value_coef, float clip_eps) {
    return critic_grad_value(values[b], clipped ? old_values[b] : 0.0f, returns[b], mb, convention, clipped, value_coef,
                             clip_eps);
}

}  // namespace mrl
