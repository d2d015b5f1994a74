/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C, single-threaded restatement of the bandwidth-bound element-wise and
 * normalisation functions that sit next to attention in a GPT-NeoX transformer
 * layer: bias + tanh-GeLU (forward, backward), bias + dropout + residual add in
 * both forms (dropout off; dropout active with a counter-based mask), gated
 * MLP activations, LayerNorm and RMSNorm (forward, backward). Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
 * leg may load this library, and only as the checker.
 *
 * Arithmetic: what the reference's fused (TorchScript) kernels and torch's
 * normalisation kernels do for 16-bit tensors -- operands are widened to fp32,
 * the whole expression is evaluated in fp32 in source order (no fused
 * multiply-add: build with -ffp-contract=off) and the result is rounded once,
 * to nearest even, to the storage type. Eager 16-bit torch rounds after every
 * operator instead; tests bound that difference separately.
 *
 * How these functions are pinned (tests/test_oracle_layer.py): float64
 * evaluation of the closed forms, torch's own library routines
 * (gelu(approximate="tanh"), layer_norm, autograd in float64), invariants
 * (normalised rows have zero mean / unit mean square, gradients are orthogonal
 * to the directions the normalisation removes), special values. The dropout
 * mask is this build's own definition (Philox4x32-10, pinned by its published
 * known-answer vectors and statistically); which elements torch's generator
 * would drop for the same seed is a different set: that part is PARITY
 * UNPINNED against the reference by construction.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#include "storage_formats.h"

/* ------------------------------------------------------------------------ */
/* bias + GeLU (tanh form)                                                    */
/* ------------------------------------------------------------------------ */

/* tanh argument of megatron/model/activations.py:81-82, in source order */
static float gelu_inner(float x)
{
    const float a = 0.044715f * x;
    const float b = a * x;
    const float c = 1.0f + b;
    const float d = 0.79788456f * x;
    return d * c;
}

/*
 * bias_gelu (megatron/model/activations.py:79-82):
 *   x = bias + y;  out = x * 0.5 * (1.0 + tanh(0.79788456 * x * (1 + 0.044715 * x * x)))
 * y, out: [rows, cols]; bias: [cols] or NULL (no bias).
 */
int oracle_bias_gelu_fwd(void* out, const void* y, const void* bias, int64_t rows, int64_t cols, int dt)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float x = load_elem(y, r * cols + c, dt);
            if (bias) x = load_elem(bias, c, dt) + x;
            const float t = tanhf(gelu_inner(x));
            const float h = x * 0.5f;
            store_elem(out, r * cols + c, dt, h * (1.0f + t));
        }
    return 0;
}

/*
 * bias_gelu_back (megatron/model/activations.py:88-97):
 *   t  = tanh(0.79788456 * x * (1 + 0.044715 * x * x))
 *   ff = 0.5 * x * ((1 - t * t) * (0.79788456 + 0.1070322243 * x * x)) + 0.5 * (1 + t)
 *   dx = ff * g
 */
int oracle_bias_gelu_bwd(void* dx, const void* g, const void* y, const void* bias, int64_t rows, int64_t cols,
                         int dt)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float x = load_elem(y, r * cols + c, dt);
            if (bias) x = load_elem(bias, c, dt) + x;
            const float t = tanhf(gelu_inner(x));
            const float sech2 = 1.0f - t * t;
            const float poly = 0.79788456f + (0.1070322243f * x) * x;
            const float left = (0.5f * x) * (sech2 * poly);
            const float right = 0.5f * (1.0f + t);
            const float ff = left + right;
            store_elem(dx, r * cols + c, dt, ff * load_elem(g, r * cols + c, dt));
        }
    return 0;
}

/*
 * Gradient of the bias: GeLUFunction.backward returns the [rows, cols] tensor
 * for both inputs (megatron/model/activations.py:108-112) and autograd reduces
 * it to the bias shape, i.e. the column sums of the *stored* dx, accumulated in
 * fp32 and rounded to the storage type.
 */
int oracle_column_sum(void* out, const void* dx, int64_t rows, int64_t cols, int dt)
{
    float* col = (float*)malloc(sizeof(float) * (size_t)(rows > 0 ? rows : 1));
    if (!col) return -2;
    for (int64_t c = 0; c < cols; ++c) {
        for (int64_t r = 0; r < rows; ++r) col[r] = load_elem(dx, r * cols + c, dt);
        store_elem(out, c, dt, pairwise_sum(col, rows));
    }
    free(col);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* bias + dropout + residual add with dropout off                            */
/* ------------------------------------------------------------------------ */

/*
 * bias_dropout_add (megatron/model/fused_bias_dropout.py:28-35) when
 * training is False or prob is 0 (torch's dropout is then the identity):
 *   out = residual + (x + bias)
 * x, residual, out: [rows, cols]; bias: [cols] or NULL; residual may be NULL
 * (:33-34).
 */
int oracle_bias_add_residual(void* out, const void* x, const void* bias, const void* residual, int64_t rows,
                             int64_t cols, int dt)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            float v = load_elem(x, r * cols + c, dt);
            if (bias) v = v + load_elem(bias, c, dt);
            if (residual) v = load_elem(residual, r * cols + c, dt) + v;
            store_elem(out, r * cols + c, dt, v);
        }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* LayerNorm and RMSNorm                                                      */
/* ------------------------------------------------------------------------ */

static float load_param(const void* p, int64_t i, int pdt) { return p ? load_elem(p, i, pdt) : 0.0f; }

/*
 * torch.nn.LayerNorm, which megatron/model/norms.py:16,32 hands out for
 * norm = "layernorm" (used as input_layernorm / post_attention_layernorm,
 * megatron/model/transformer.py:985-1040): per row of `cols` elements
 *   mean = sum(x) / cols, var = sum((x - mean)^2) / cols (biased),
 *   rstd = 1 / sqrt(var + eps), y = ((x - mean) * rstd) * gamma + beta,
 * statistics and arithmetic in fp32 whatever the storage type, y rounded once.
 * gamma / beta: [cols] in storage type pdt (fp32 or the type of x), or NULL
 * (no affine term). mean, rstd: fp32 [rows], what the backward needs.
 */
int oracle_layernorm_fwd(void* y, float* mean, float* rstd, const void* x, const void* gamma, const void* beta,
                         float eps, int64_t rows, int64_t cols, int dt, int pdt)
{
    float* v = (float*)malloc(sizeof(float) * (size_t)(cols > 0 ? cols : 1));
    if (!v) return -2;
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t c = 0; c < cols; ++c) v[c] = load_elem(x, r * cols + c, dt);
        const float m = pairwise_sum(v, cols) / (float)cols;
        for (int64_t c = 0; c < cols; ++c) {
            const float d = v[c] - m;
            v[c] = d * d;
        }
        const float var = pairwise_sum(v, cols) / (float)cols;
        const float rs = 1.0f / sqrtf(var + eps);
        for (int64_t c = 0; c < cols; ++c) {
            float o = (load_elem(x, r * cols + c, dt) - m) * rs;
            if (gamma) o = o * load_param(gamma, c, pdt);
            if (beta) o = o + load_param(beta, c, pdt);
            store_elem(y, r * cols + c, dt, o);
        }
        if (mean) mean[r] = m;
        if (rstd) rstd[r] = rs;
    }
    free(v);
    return 0;
}

/*
 * Backward of the above (the textbook adjoint, as torch's layer_norm backward):
 *   xhat = (x - mean) * rstd, g = dy * gamma,
 *   dx = rstd * (g - (sum(g) + xhat * sum(g * xhat)) / cols),
 *   dgamma[c] = sum over rows of dy * xhat, dbeta[c] = sum over rows of dy,
 * fp32 throughout, outputs rounded once (dgamma, dbeta to pdt). Any of dx,
 * dgamma, dbeta may be NULL.
 */
static int layernorm_dx(void* dx, const void* dy, const void* dy2, const void* x, const float* mean,
                        const float* rstd, const void* gamma, const void* gamma2, int64_t rows, int64_t cols, int dt,
                        int pdt);

int oracle_layernorm_bwd(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x, const float* mean,
                         const float* rstd, const void* gamma, int64_t rows, int64_t cols, int dt, int pdt)
{
    const size_t n = (size_t)(cols > 0 ? cols : 1);
    float* g = (float*)malloc(sizeof(float) * n);
    float* gx = (float*)malloc(sizeof(float) * n);
    float* col = (float*)malloc(sizeof(float) * (size_t)(rows > 0 ? rows : 1));
    if (!g || !gx || !col) {
        free(g);
        free(gx);
        free(col);
        return -2;
    }
    if (dx)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t c = 0; c < cols; ++c) {
                const float xh = (load_elem(x, r * cols + c, dt) - mean[r]) * rstd[r];
                g[c] = load_elem(dy, r * cols + c, dt) * (gamma ? load_param(gamma, c, pdt) : 1.0f);
                gx[c] = g[c] * xh;
            }
            const float s1 = pairwise_sum(g, cols), s2 = pairwise_sum(gx, cols);
            for (int64_t c = 0; c < cols; ++c) {
                const float xh = (load_elem(x, r * cols + c, dt) - mean[r]) * rstd[r];
                const float t = (s1 + xh * s2) / (float)cols;
                store_elem(dx, r * cols + c, dt, rstd[r] * (g[c] - t));
            }
        }
    for (int64_t c = 0; c < cols; ++c) {
        if (dgamma) {
            for (int64_t r = 0; r < rows; ++r)
                col[r] = load_elem(dy, r * cols + c, dt) * ((load_elem(x, r * cols + c, dt) - mean[r]) * rstd[r]);
            store_elem(dgamma, c, pdt, pairwise_sum(col, rows));
        }
        if (dbeta) {
            for (int64_t r = 0; r < rows; ++r) col[r] = load_elem(dy, r * cols + c, dt);
            store_elem(dbeta, c, pdt, pairwise_sum(col, rows));
        }
    }
    free(g);
    free(gx);
    free(col);
    return 0;
}

/*
 * RMSNorm and ScaleNorm. Three definitions live in the reference, selected here by eps_mode:
 *   1: the Python class RMSNorm, megatron/model/norms.py:54-107:
 *        rms = ||x[:stat]||_2 * stat^(-1/2);  y = scale * (x / (rms + eps)) [+ offset]
 *      stat = cols, or int(cols * p) leading columns for the partial variant (:87-94)
 *   0: the fused variants (MixedFusedRMSNorm, megatron/model/fused_layer_norm.py:156-252,
 *      backed by apex, and TERMSNorm): y = scale * (x * rsqrt(mean(x^2) + eps))
 *   2: ScaleNorm, megatron/model/norms.py:110-119: y = x / max(||x||_2, eps) * g; the
 *      scalar g arrives as a scale vector of equal values
 * fp32 arithmetic, one rounding of y. inv: fp32 [rows], the factor x is
 * multiplied by.
 */
static float rms_inverse(float sumsq, int64_t stat, float eps, int eps_mode)
{
    if (eps_mode == 2) {
        const float nrm = sqrtf(sumsq);
        return 1.0f / (nrm > eps ? nrm : eps);
    }
    if (eps_mode == 1) return 1.0f / (sqrtf(sumsq) * (1.0f / sqrtf((float)stat)) + eps);
    return 1.0f / sqrtf(sumsq / (float)stat + eps);
}

int oracle_rmsnorm_fwd(void* y, float* inv, const void* x, const void* scale, const void* offset, float eps,
                       int eps_mode, int64_t rows, int64_t cols, int64_t stat, int dt, int pdt)
{
    float* v = (float*)malloc(sizeof(float) * (size_t)(cols > 0 ? cols : 1));
    if (!v) return -2;
    if (stat < 1 || stat > cols) {
        free(v);
        return -1;
    }
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t c = 0; c < stat; ++c) {
            const float f = load_elem(x, r * cols + c, dt);
            v[c] = f * f;
        }
        const float iv = rms_inverse(pairwise_sum(v, stat), stat, eps, eps_mode);
        for (int64_t c = 0; c < cols; ++c) {
            float o = load_elem(x, r * cols + c, dt) * iv;
            if (scale) o = load_param(scale, c, pdt) * o;
            if (offset) o = o + load_param(offset, c, pdt);
            store_elem(y, r * cols + c, dt, o);
        }
        if (inv) inv[r] = iv;
    }
    free(v);
    return 0;
}

/*
 * Backward of RMSNorm: with xhat = x * inv, g = dy * scale, s = sum over all columns of g * xhat,
 * and m[c] = 1 for the columns c < stat the statistic was taken over, else 0:
 *   eps_mode 0: dx = inv * (g - m * xhat * s / stat)
 *   eps_mode 1: dx = inv * (g - m * xhat * s / (stat * rho)), rho = rms / (rms + eps) = 1 - eps * inv
 *               (rho = 0, an all-zero row with eps > 0: the second term is 0, as
 *               torch's norm backward defines it)
 *   eps_mode 2: dx = inv * (g - xhat * s) while ||x|| > eps (inv < 1 / eps); a clamped norm
 *               is a constant: dx = inv * g
 *   dscale[c] = sum over rows of dy * xhat, doffset[c] = sum over rows of dy.
 */
int oracle_rmsnorm_bwd(void* dx, void* dscale, void* doffset, const void* dy, const void* x, const float* inv,
                       const void* scale, float eps, int eps_mode, int64_t rows, int64_t cols, int64_t stat, int dt,
                       int pdt)
{
    if (stat < 1 || stat > cols) return -1;
    const size_t n = (size_t)(cols > 0 ? cols : 1);
    float* g = (float*)malloc(sizeof(float) * n);
    float* gx = (float*)malloc(sizeof(float) * n);
    float* col = (float*)malloc(sizeof(float) * (size_t)(rows > 0 ? rows : 1));
    if (!g || !gx || !col) {
        free(g);
        free(gx);
        free(col);
        return -2;
    }
    if (dx)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t c = 0; c < cols; ++c) {
                const float xh = load_elem(x, r * cols + c, dt) * inv[r];
                g[c] = load_elem(dy, r * cols + c, dt) * (scale ? load_param(scale, c, pdt) : 1.0f);
                gx[c] = g[c] * xh;
            }
            const float s = pairwise_sum(gx, cols);
            float k = s / (float)stat;
            if (eps_mode == 1) {
                const float rho = 1.0f - eps * inv[r];
                k = rho > 0.0f ? k / rho : 0.0f;
            } else if (eps_mode == 2) {
                k = inv[r] < 1.0f / eps ? s : 0.0f;
            }
            for (int64_t c = 0; c < cols; ++c) {
                const float xh = load_elem(x, r * cols + c, dt) * inv[r];
                const float t = c < stat ? xh * k : 0.0f;
                store_elem(dx, r * cols + c, dt, inv[r] * (g[c] - t));
            }
        }
    for (int64_t c = 0; c < cols; ++c) {
        if (dscale) {
            for (int64_t r = 0; r < rows; ++r)
                col[r] = load_elem(dy, r * cols + c, dt) * (load_elem(x, r * cols + c, dt) * inv[r]);
            store_elem(dscale, c, pdt, pairwise_sum(col, rows));
        }
        if (doffset) {
            for (int64_t r = 0; r < rows; ++r) col[r] = load_elem(dy, r * cols + c, dt);
            store_elem(doffset, c, pdt, pairwise_sum(col, rows));
        }
    }
    free(g);
    free(gx);
    free(col);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* gated MLP activations                                                      */
/* ------------------------------------------------------------------------ */

enum { GATE_SWISH = 0, GATE_GELU = 1, GATE_RELU = 2, GATE_SIGMOID = 3, GATE_IDENTITY = 4 };

static float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }

/* act(g) for the activation functions get_activation pairs with a gate
 * (megatron/model/activations.py:30-49): swish = x * sigmoid(x) (:128-130),
 * F.gelu (erf form), F.relu, F.sigmoid, identity; and its derivative. */
static void gate_eval(int act, float g, float* a, float* da)
{
    switch (act) {
    case GATE_SWISH: {
        const float s = sigmoid_f(g);
        *a = g * s;
        *da = s * (1.0f + g * (1.0f - s));
        break;
    }
    case GATE_GELU: {
        const float cdf = 0.5f * (1.0f + erff(g * 0.70710678118654752f));
        const float pdf = 0.3989422804014327f * expf(-0.5f * g * g);
        *a = g * cdf;
        *da = cdf + g * pdf;
        break;
    }
    case GATE_RELU:
        *a = g > 0.0f ? g : 0.0f;
        *da = g > 0.0f ? 1.0f : 0.0f;
        break;
    case GATE_SIGMOID: {
        const float s = sigmoid_f(g);
        *a = s;
        *da = s * (1.0f - s);
        break;
    }
    default:
        *a = g;
        *da = 1.0f;
    }
}

/*
 * Gated_Activation.forward (megatron/model/transformer.py:192-206):
 *   x, gate = in.chunk(2, dim=-1); with a bias, x += bias_1, gate += bias_2;
 *   out = activation_func(gate) * x
 * in: [rows, 2f], bias: [2f] or NULL, out: [rows, f].
 */
int oracle_gated_act_fwd(void* out, const void* in, const void* bias, int64_t rows, int64_t f, int act, int dt)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < f; ++c) {
            float x = load_elem(in, r * 2 * f + c, dt);
            float g = load_elem(in, r * 2 * f + f + c, dt);
            if (bias) {
                x = x + load_elem(bias, c, dt);
                g = g + load_elem(bias, f + c, dt);
            }
            float a, da;
            gate_eval(act, g, &a, &da);
            store_elem(out, r * f + c, dt, a * x);
        }
    return 0;
}

/* Its adjoint (the reference leaves it to autograd): din = (dy * act(g), dy * x * act'(g)). */
int oracle_gated_act_bwd(void* din, const void* dy, const void* in, const void* bias, int64_t rows, int64_t f,
                         int act, int dt)
{
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < f; ++c) {
            float x = load_elem(in, r * 2 * f + c, dt);
            float g = load_elem(in, r * 2 * f + f + c, dt);
            if (bias) {
                x = x + load_elem(bias, c, dt);
                g = g + load_elem(bias, f + c, dt);
            }
            float a, da;
            gate_eval(act, g, &a, &da);
            const float d = load_elem(dy, r * f + c, dt);
            store_elem(din, r * 2 * f + c, dt, d * a);
            store_elem(din, r * 2 * f + f + c, dt, (d * x) * da);
        }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* bias + dropout + residual add with dropout active                         */
/* ------------------------------------------------------------------------ */

/* Philox4x32-10 (Salmon, Moraes, Dror, Shaw: "Parallel random numbers: as easy
 * as 1, 2, 3", SC'11; the generator family torch's CUDA dropout draws from). */
void oracle_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = counter[0], c1 = counter[1], c2 = counter[2], c3 = counter[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c0 = n0;
        c1 = (uint32_t)p1;
        c2 = n2;
        c3 = (uint32_t)p0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

/* keep[e] for e in [0, n): 16 bits per element, eight elements per Philox call
 * with counter (e / 8, offset) and key seed; kept when below round((1 - p) * 65536). */
int oracle_dropout_mask(uint8_t* keep, int64_t n, float p, uint64_t seed, uint64_t offset)
{
    const double kp = 1.0 - (double)p;
    uint32_t threshold = (uint32_t)(kp * 65536.0 + 0.5);
    if (threshold > 65536u) threshold = 65536u;
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    for (int64_t g = 0; g * 8 < n; ++g) {
        const uint32_t ctr[4] = {(uint32_t)g, (uint32_t)((uint64_t)g >> 32), (uint32_t)offset, (uint32_t)(offset >> 32)};
        uint32_t r[4];
        oracle_philox4x32_10(ctr, key, r);
        for (int j = 0; j < 8 && g * 8 + j < n; ++j) {
            const uint32_t v = (r[j >> 1] >> ((j & 1) * 16)) & 0xffffu;
            keep[g * 8 + j] = v < threshold;
        }
    }
    return 0;
}

/*
 * bias_dropout_add (megatron/model/fused_bias_dropout.py:28-35) with training
 * True and 0 < prob < 1: out = residual + dropout(x + bias), dropout(v) = keep ?
 * v / (1 - p) : 0 (torch.nn.functional.dropout), here with the mask above,
 * fp32 arithmetic and one rounding. x == NULL is not allowed; bias, residual
 * may be NULL. With residual == NULL and bias == NULL this is the backward of
 * the dropout applied to x = grad.
 */
int oracle_bias_dropout_add(void* out, const void* x, const void* bias, const void* residual, int64_t rows,
                            int64_t cols, float p, uint64_t seed, uint64_t offset, int dt)
{
    const int64_t n = rows * cols;
    uint8_t* keep = (uint8_t*)malloc((size_t)(n > 0 ? n : 1));
    if (!keep) return -2;
    oracle_dropout_mask(keep, n, p, seed, offset);
    const float scale = (float)(1.0 / (1.0 - (double)p));
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t c = 0; c < cols; ++c) {
            const int64_t e = r * cols + c;
            float v = load_elem(x, e, dt);
            if (bias) v = v + load_elem(bias, c, dt);
            v = keep[e] ? v * scale : 0.0f;
            if (residual) v = load_elem(residual, e, dt) + v;
            store_elem(out, e, dt, v);
        }
    free(keep);
    return 0;
}

/*
 * Two LayerNorms of one input (the parallel-residual layer applies input_layernorm and
 * post_attention_layernorm to the same x, megatron/model/transformer.py:1195-1213): the statistics are shared,
 * and since the backward is linear in g the gradient with respect to x is the single formula above with
 *   g = dy1 * gamma1 + dy2 * gamma2
 * evaluated in fp32 and rounded once (autograd would round each dx and add them: up to 1.5 ulp more).
 * The parameter gradients are those of the two single calls.
 */
static int layernorm_dx(void* dx, const void* dy, const void* dy2, const void* x, const float* mean,
                        const float* rstd, const void* gamma, const void* gamma2, int64_t rows, int64_t cols, int dt,
                        int pdt)
{
    const size_t n = (size_t)(cols > 0 ? cols : 1);
    float* g = (float*)malloc(sizeof(float) * n);
    float* gx = (float*)malloc(sizeof(float) * n);
    if (!g || !gx) {
        free(g);
        free(gx);
        return -2;
    }
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t c = 0; c < cols; ++c) {
            const float xh = (load_elem(x, r * cols + c, dt) - mean[r]) * rstd[r];
            g[c] = load_elem(dy, r * cols + c, dt) * (gamma ? load_param(gamma, c, pdt) : 1.0f);
            if (dy2) g[c] = g[c] + load_elem(dy2, r * cols + c, dt) * (gamma2 ? load_param(gamma2, c, pdt) : 1.0f);
            gx[c] = g[c] * xh;
        }
        const float s1 = pairwise_sum(g, cols), s2 = pairwise_sum(gx, cols);
        for (int64_t c = 0; c < cols; ++c) {
            const float xh = (load_elem(x, r * cols + c, dt) - mean[r]) * rstd[r];
            const float t = (s1 + xh * s2) / (float)cols;
            store_elem(dx, r * cols + c, dt, rstd[r] * (g[c] - t));
        }
    }
    free(g);
    free(gx);
    return 0;
}

int oracle_layernorm_pair_dx(void* dx, const void* dy1, const void* dy2, const void* x, const float* mean,
                             const float* rstd, const void* gamma1, const void* gamma2, int64_t rows, int64_t cols,
                             int dt, int pdt)
{
    return layernorm_dx(dx, dy1, dy2, x, mean, rstd, gamma1, gamma2, rows, cols, dt, pdt);
}
