/*
 * MLP layers: CPU restatement (test infrastructure, never shipped).
 *
 *   Linear            deep_rl/model/linear.mojo:41-121 (forward), :990-1049 (backward)
 *   LinearReLU        deep_rl/model/linear_relu.mojo:49-135, backward with ReLU mask
 *   LinearTanh        deep_rl/model/linear_tanh.mojo:48-127 (forward), :726-784 (backward)
 *   StochasticActor   deep_rl/model/stochastic_actor.mojo:197-299 (Float64 accumulation),
 *                     :305-378 (backward)
 *   Seq2 chaining     deep_rl/model/sequential.mojo:85-143 (params [L0|L1|...],
 *                     cache blocked per layer [BATCH x CACHE_i])
 *
 * Parameters of a layer: W row-major [in, out] then b [out] (actor head: W_mean,
 * b_mean, log_std).  Accumulation order: bias first, then k ascending, fp32.
 * backward ACCUMULATES into grads like the CPU reference; callers zero grads first,
 * which is also what makes it equal to the GPU path's overwrite semantics.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include "orc.h"

int orc_layer_out_dim(const orc_layer *l) {
    return l->kind == ORC_STOCHASTIC_ACTOR ? 2 * l->out_dim : l->out_dim;
}
int orc_layer_param_size(const orc_layer *l) {
    int p = l->in_dim * l->out_dim + l->out_dim;
    return l->kind == ORC_STOCHASTIC_ACTOR ? p + l->out_dim : p;
}
int orc_layer_cache_size(const orc_layer *l) {
    if (l->kind == ORC_LINEAR || l->kind == ORC_STOCHASTIC_ACTOR) return l->in_dim;
    return l->in_dim + l->out_dim;
}
int orc_mlp_param_size(const orc_layer *ls, int n) {
    int s = 0;
    for (int i = 0; i < n; ++i) s += orc_layer_param_size(ls + i);
    return s;
}
int orc_mlp_cache_size(const orc_layer *ls, int n) {
    int s = 0;
    for (int i = 0; i < n; ++i) s += orc_layer_cache_size(ls + i);
    return s;
}

static void layer_forward(const orc_layer *l, int batch, const float *in, const float *params,
                          float *out, float *cache) {
    const int I = l->in_dim, O = l->out_dim;
    const int CS = orc_layer_cache_size(l);
    const float *W = params, *b = params + I * O;
    if (l->kind == ORC_STOCHASTIC_ACTOR) {
        const float *log_std = b + O;
        for (int n = 0; n < batch; ++n) {
            if (cache) memcpy(cache + (long)n * CS, in + (long)n * I, sizeof(float) * I);
            for (int j = 0; j < O; ++j) {
                double acc = (double)b[j];
                for (int i = 0; i < I; ++i) acc += (double)in[(long)n * I + i] * (double)W[i * O + j];
                out[(long)n * 2 * O + j] = (float)acc;
            }
            for (int j = 0; j < O; ++j) {
                double v = (double)log_std[j];
                if (v < -5.0) v = -5.0;
                else if (v > 2.0) v = 2.0;
                out[(long)n * 2 * O + O + j] = (float)v;
            }
        }
        return;
    }
    for (int n = 0; n < batch; ++n) {
        const float *x = in + (long)n * I;
        if (cache) memcpy(cache + (long)n * CS, x, sizeof(float) * I);
        for (int j = 0; j < O; ++j) {
            float acc = b[j];
            for (int i = 0; i < I; ++i) acc += x[i] * W[i * O + j];
            float y = acc;
            if (l->kind == ORC_LINEAR_RELU) {
                if (cache) cache[(long)n * CS + I + j] = acc; /* pre-activation */
                y = acc > 0.0f ? acc : 0.0f;
            } else if (l->kind == ORC_LINEAR_TANH) {
                y = tanhf(acc);
                if (cache) cache[(long)n * CS + I + j] = y; /* tanh output */
            }
            out[(long)n * O + j] = y;
        }
    }
}

void orc_mlp_forward(const orc_layer *ls, int n, int batch, const float *in, const float *params,
                     float *out, float *cache) {
    const float *cur = in;
    float *tmp_a = 0;
    for (int k = 0; k < n; ++k) {
        int od = orc_layer_out_dim(ls + k);
        float *dst = (k == n - 1) ? out : (float *)malloc(sizeof(float) * (size_t)batch * od);
        layer_forward(ls + k, batch, cur, params, dst, cache);
        params += orc_layer_param_size(ls + k);
        if (cache) cache += (long)batch * orc_layer_cache_size(ls + k);
        if (tmp_a) free(tmp_a);
        tmp_a = (k == n - 1) ? 0 : dst;
        cur = dst;
    }
}

static void layer_backward(const orc_layer *l, int batch, const float *gout, const float *params,
                           const float *cache, float *grads, float *gin) {
    const int I = l->in_dim, O = l->out_dim;
    const int CS = orc_layer_cache_size(l);
    const float *W = params;
    float *dW = grads, *db = grads + I * O;
    if (l->kind == ORC_STOCHASTIC_ACTOR) {
        float *dls = db + O;
        for (int n = 0; n < batch; ++n) {
            const float *g = gout + (long)n * 2 * O;
            const float *x = cache + (long)n * CS;
            if (gin) {
                for (int i = 0; i < I; ++i) {
                    float acc = 0.0f;
                    for (int j = 0; j < O; ++j) acc = acc + g[j] * W[i * O + j];
                    gin[(long)n * I + i] = acc;
                }
            }
            for (int i = 0; i < I; ++i)
                for (int j = 0; j < O; ++j) dW[i * O + j] = dW[i * O + j] + x[i] * g[j];
            for (int j = 0; j < O; ++j) db[j] = db[j] + g[j];
            for (int j = 0; j < O; ++j) dls[j] = dls[j] + g[O + j];
        }
        return;
    }
    float *m = (float *)malloc(sizeof(float) * (size_t)O);
    for (int n = 0; n < batch; ++n) {
        const float *g = gout + (long)n * O;
        const float *c = cache + (long)n * CS;
        for (int j = 0; j < O; ++j) {
            if (l->kind == ORC_LINEAR_RELU) m[j] = c[I + j] > 0.0f ? g[j] : 0.0f;
            else if (l->kind == ORC_LINEAR_TANH) m[j] = g[j] * (1.0f - c[I + j] * c[I + j]);
            else m[j] = g[j];
        }
        if (gin) {
            for (int i = 0; i < I; ++i) {
                float acc = 0.0f;
                for (int j = 0; j < O; ++j) acc += m[j] * W[i * O + j];
                gin[(long)n * I + i] = acc;
            }
        }
        for (int i = 0; i < I; ++i)
            for (int j = 0; j < O; ++j) dW[i * O + j] = dW[i * O + j] + c[i] * m[j];
        for (int j = 0; j < O; ++j) db[j] = db[j] + m[j];
    }
    free(m);
}

void orc_mlp_backward(const orc_layer *ls, int n, int batch, const float *grad_out,
                      const float *params, const float *cache, float *grads, float *grad_in) {
    /* locate each layer's slices */
    long poff[16], coff[16];
    long p = 0, c = 0;
    for (int k = 0; k < n; ++k) {
        poff[k] = p; coff[k] = c;
        p += orc_layer_param_size(ls + k);
        c += (long)batch * orc_layer_cache_size(ls + k);
    }
    const float *g = grad_out;
    float *owned = 0;
    for (int k = n - 1; k >= 0; --k) {
        float *gin;
        if (k == 0) gin = grad_in;
        else gin = (float *)malloc(sizeof(float) * (size_t)batch * ls[k].in_dim);
        layer_backward(ls + k, batch, g, params + poff[k], cache + coff[k], grads + poff[k], gin);
        if (owned) free(owned);
        owned = (k == 0) ? 0 : gin;
        g = gin;
    }
}
