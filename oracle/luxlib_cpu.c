/*
 * CPU restatement, in plain C, of LuxLib's LoopedArrayOp (CPU) path for the operators of the
 * benchmarked chain: batchnorm (training) -> bias_activation, forward and pullback.
 *
 * TEST INFRASTRUCTURE ONLY: this is the timed "cpu_baseline" (kind "port") of the benchmark
 * and a cross-check of the numpy oracle.  It is never linked into the product library.
 *
 * The loop structure and threading follow the reference (paths relative to
 * lib/LuxLib/src/impl/): statistics are serial reductions (Statistics.mean / var,
 * common_ops.jl:40-43), the normalise loop is threaded over the batch dimension only
 * (batchnorm.jl:212-227, Threads.@threads), bias_activation, the activation gradient, the
 * bias gradient and the fused batchnorm backward loop are serial @simd loops
 * (bias_activation.jl:253-270, activation.jl:142-154, common_ops.jl:34-38,
 * batchnorm.jl:517-570), and the mean_var pullback is a broadcast (common_ops.jl:45-61).
 * All tensors are fp32, column-major (I, C, N).
 *
 * Pinned by tests/test_oracle_c.py against the numpy oracle (itself pinned by the reference's
 * known-answer tests and torch autograd) and the batchnorm known-answer test directly.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ACT_IDENTITY 0
#define ACT_RELU 1
#define ACT_TANH 2
#define ACT_SIGMOID 3
#define ACT_SWISH 4
#define ACT_GELU 5

static inline float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

static inline float act_f(int act, float x) {
    switch (act) {
        case ACT_RELU: return x > 0.0f ? x : 0.0f;
        case ACT_TANH: return tanhf(x);
        case ACT_SIGMOID: return sigmoidf_(x);
        case ACT_SWISH: return x * sigmoidf_(x);
        case ACT_GELU: {
            float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
            return 0.5f * x * (1.0f + tanhf(u));
        }
        default: return x;
    }
}

/* derivative given the output o and the pre-activation x (utils.jl:81-84) */
static inline float act_d(int act, float o, float x) {
    switch (act) {
        case ACT_RELU: return o > 0.0f ? 1.0f : 0.0f;
        case ACT_TANH: return 1.0f - o * o;
        case ACT_SIGMOID: return o * (1.0f - o);
        case ACT_SWISH: return o + sigmoidf_(x) * (1.0f - o);
        case ACT_GELU: {
            float x2 = x * x;
            float u = 0.7978845608028654f * (x + 0.044715f * x2 * x);
            float t = tanhf(u);
            float du = 0.7978845608028654f * (1.0f + 3.0f * 0.044715f * x2);
            return 0.5f * (1.0f + t) + 0.5f * x * (1.0f - t * t) * du;
        }
        default: return 1.0f;
    }
}

int luxcpu_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* y[i,c,n] = act(x[i,c,n] + b[c])  -- bias_activation_simd_loop! (bias_activation.jl:253-270) */
void luxcpu_bias_activation_fwd(int act, int64_t I, int64_t C, int64_t N, const float* x, const float* b, float* y) {
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float bc = b ? b[c] : 0.0f;
            const float* xr = x + (n * C + c) * I;
            float* yr = y + (n * C + c) * I;
            for (int64_t i = 0; i < I; ++i) yr[i] = act_f(act, xr[i] + bc);
        }
}

/* dx = delta .* act'(out, pre) (activation.jl:142-154); db = sum! over all dims but C
 * (common_ops.jl:34-38).  pre may be NULL for output-only activations. */
void luxcpu_bias_activation_bwd(int act, int64_t I, int64_t C, int64_t N, const float* delta, const float* out,
                                const float* pre, float* dx, float* db) {
    const int64_t total = I * C * N;
    for (int64_t e = 0; e < total; ++e) dx[e] = act_d(act, out ? out[e] : 0.0f, pre ? pre[e] : 0.0f) * delta[e];
    if (db) {
        for (int64_t c = 0; c < C; ++c) db[c] = 0.0f;
        for (int64_t n = 0; n < N; ++n)
            for (int64_t c = 0; c < C; ++c) {
                const float* r = dx + (n * C + c) * I;
                float s = 0.0f;
                for (int64_t i = 0; i < I; ++i) s += r[i];
                db[c] += s;
            }
    }
}

/* batchnorm, training mode (batchnorm.jl:29-49,117-147,212-227; normalization.jl:20-37,95-143).
 * rmean/rvar may be NULL (then rmean_out/rvar_out are untouched). mean_out/var_out: length C. */
void luxcpu_batchnorm_train_fwd(int act, int64_t I, int64_t C, int64_t N, const float* x, const float* gamma,
                                const float* beta, const float* rmean, const float* rvar, float momentum, float eps,
                                float* y, float* rmean_out, float* rvar_out, float* mean_out, float* var_out) {
    const float cnt = (float)(I * N);
    /* mean(x; dims) then var(x; dims, corrected=false, mean) -- two serial passes */
    for (int64_t c = 0; c < C; ++c) mean_out[c] = 0.0f;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float* r = x + (n * C + c) * I;
            float s = 0.0f;
            for (int64_t i = 0; i < I; ++i) s += r[i];
            mean_out[c] += s;
        }
    for (int64_t c = 0; c < C; ++c) mean_out[c] /= cnt;
    for (int64_t c = 0; c < C; ++c) var_out[c] = 0.0f;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float* r = x + (n * C + c) * I;
            const float m = mean_out[c];
            float s = 0.0f;
            for (int64_t i = 0; i < I; ++i) s += (r[i] - m) * (r[i] - m);
            var_out[c] += s;
        }
    for (int64_t c = 0; c < C; ++c) var_out[c] /= cnt;
    if (rmean) {
        const float m1 = momentum, m2 = momentum * cnt / (cnt - 1.0f), m3 = 1.0f - momentum;
        for (int64_t c = 0; c < C; ++c) {
            rmean_out[c] = m3 * rmean[c] + m1 * mean_out[c];
            rvar_out[c] = m3 * rvar[c] + m2 * var_out[c];
        }
    }
    float* gp = (float*)malloc(sizeof(float) * (size_t)C * 2);
    float* bp = gp + C;
    for (int64_t c = 0; c < C; ++c) {
        gp[c] = (gamma ? gamma[c] : 1.0f) / sqrtf(var_out[c] + eps);
        bp[c] = (beta ? beta[c] : 0.0f) - mean_out[c] * gp[c];
    }
    /* Threads.@threads for K in axes(x, 3) */
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float* xr = x + (n * C + c) * I;
            float* yr = y + (n * C + c) * I;
            const float g = gp[c], b = bp[c];
            if (act == ACT_IDENTITY)
                for (int64_t i = 0; i < I; ++i) yr[i] = xr[i] * g + b;
            else
                for (int64_t i = 0; i < I; ++i) yr[i] = act_f(act, xr[i] * g + b);
        }
    free(gp);
}

/* Pullback w.r.t. (x, gamma, beta) for act == identity applied outside (the reference
 * differentiates the activation separately, batchnorm.jl:405-443): dy is the cotangent of the
 * affine-normalised value.  Serial fused loop (batchnorm.jl:517-570) + mean_var pullback
 * broadcast (common_ops.jl:45-61). */
void luxcpu_batchnorm_train_bwd(int64_t I, int64_t C, int64_t N, const float* dy, const float* x, const float* gamma,
                                const float* mean, const float* var, float eps, float* dx, float* dgamma,
                                float* dbeta) {
    const float cnt = (float)(I * N);
    float* dmu = (float*)calloc((size_t)C * 4, sizeof(float));
    float* dvar = dmu + C;
    float* dg = dmu + 2 * C;
    float* dbt = dmu + 3 * C;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float idenom = 1.0f / sqrtf(var[c] + eps);
            const float idenom2 = idenom * idenom;
            const float gp = (gamma ? gamma[c] : 1.0f) * idenom;
            const float* dr = dy + (n * C + c) * I;
            const float* xr = x + (n * C + c) * I;
            float* o = dx + (n * C + c) * I;
            float a_mu = 0.0f, a_var = 0.0f, a_g = 0.0f, a_b = 0.0f;
            for (int64_t i = 0; i < I; ++i) {
                const float xmu = xr[i] - mean[c];
                o[i] = dr[i] * gp;
                a_mu -= o[i];
                a_var -= o[i] * xmu * 0.5f * idenom2;
                a_g += dr[i] * xmu * idenom;
                a_b += dr[i];
            }
            dmu[c] += a_mu; dvar[c] += a_var; dg[c] += a_g; dbt[c] += a_b;
        }
    /* mean_var rrule: dx += dmu / n + (2 / n) * dvar * (x - mu) */
    for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < C; ++c) {
            const float* xr = x + (n * C + c) * I;
            float* o = dx + (n * C + c) * I;
            const float a = dmu[c] / cnt, b = (2.0f / cnt) * dvar[c], m = mean[c];
            for (int64_t i = 0; i < I; ++i) o[i] += a + b * (xr[i] - m);
        }
    if (dgamma) memcpy(dgamma, dg, sizeof(float) * (size_t)C);
    if (dbeta) memcpy(dbeta, dbt, sizeof(float) * (size_t)C);
    free(dmu);
}

/* groupnorm (groupnorm.jl:5-22): x viewed as (I, Cg, G, N); statistics per (group, sample) as two
 * serial passes (mean, then var about it, common_ops.jl:40-43); the affine-normalise loop
 * (groupnorm_affine_normalize_act_cpu!, groupnorm.jl:131-205) is a serial @simd loop, as is its
 * pullback (:477-533): nothing here is threaded, as in the reference.  mean/var: (G, N). */
void luxcpu_groupnorm_fwd(int act, int64_t I, int64_t Cg, int64_t G, int64_t N, const float* x, const float* gamma,
                          const float* beta, float eps, float* y, float* mean, float* var) {
    const int64_t m = I * Cg;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < G; ++k) {
            const float* xs = x + (n * G + k) * m;
            float s = 0.0f;
            for (int64_t e = 0; e < m; ++e) s += xs[e];
            const float mu = s / (float)m;
            float d = 0.0f;
            for (int64_t e = 0; e < m; ++e) d += (xs[e] - mu) * (xs[e] - mu);
            mean[n * G + k] = mu;
            var[n * G + k] = d / (float)m;
        }
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < G; ++k) {
            const float idenom = 1.0f / sqrtf(var[n * G + k] + eps);
            const float mu = mean[n * G + k];
            for (int64_t j = 0; j < Cg; ++j) {
                const int64_t c = k * Cg + j;
                const float sc = (gamma ? gamma[c] : 1.0f) * idenom;
                const float sh = (beta ? beta[c] : 0.0f) - mu * sc;
                const float* xr = x + ((n * G + k) * Cg + j) * I;
                float* yr = y + ((n * G + k) * Cg + j) * I;
                for (int64_t i = 0; i < I; ++i) yr[i] = act_f(act, xr[i] * sc + sh);
            }
        }
}

/* Pullback of the same w.r.t. (x, gamma, beta): the activation's derivative from the recomputed
 * pre-activation (the rrule keeps it, groupnorm.jl:349-404), the fused loop (:477-533) and the
 * mean_var pullback broadcast (common_ops.jl:45-61). */
void luxcpu_groupnorm_bwd(int act, int64_t I, int64_t Cg, int64_t G, int64_t N, const float* delta, const float* x,
                          const float* gamma, const float* beta, const float* mean, const float* var, float eps,
                          float* dx, float* dgamma, float* dbeta) {
    const int64_t m = I * Cg, C = Cg * G;
    if (dgamma) for (int64_t c = 0; c < C; ++c) dgamma[c] = 0.0f;
    if (dbeta) for (int64_t c = 0; c < C; ++c) dbeta[c] = 0.0f;
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < G; ++k) {
            const float mu = mean[n * G + k];
            const float idenom = 1.0f / sqrtf(var[n * G + k] + eps);
            const float idenom2 = idenom * idenom;
            float dmu = 0.0f, dvar = 0.0f;
            for (int64_t j = 0; j < Cg; ++j) {
                const int64_t c = k * Cg + j;
                const float g = gamma ? gamma[c] : 1.0f, b = beta ? beta[c] : 0.0f;
                const float sc = g * idenom, sh = b - mu * sc;
                const float* xr = x + ((n * G + k) * Cg + j) * I;
                const float* dr = delta + ((n * G + k) * Cg + j) * I;
                float* o = dx + ((n * G + k) * Cg + j) * I;
                float ag = 0.0f, ab = 0.0f;
                for (int64_t i = 0; i < I; ++i) {
                    const float pre = xr[i] * sc + sh;
                    const float dy = dr[i] * act_d(act, act_f(act, pre), pre);
                    const float xmu = xr[i] - mu;
                    o[i] = dy * sc;
                    dmu -= o[i];
                    dvar -= o[i] * xmu * 0.5f * idenom2;
                    ag += dy * xmu * idenom;
                    ab += dy;
                }
                if (dgamma) dgamma[c] += ag;
                if (dbeta) dbeta[c] += ab;
            }
            const float a = dmu / (float)m, bb = (2.0f / (float)m) * dvar;
            for (int64_t e = 0; e < m; ++e) {
                float* o = dx + (n * G + k) * m;
                o[e] += a + bb * (x[(n * G + k) * m + e] - mu);
            }
        }
}
