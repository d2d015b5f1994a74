/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C, single-threaded restatement of the bandwidth-bound element-wise and
 * normalisation functions that sit next to attention in a GPT-NeoX transformer
 * layer: bias + tanh-GeLU (forward, backward), bias + dropout + residual add in
 * its deterministic form (dropout off), LayerNorm and RMSNorm (forward,
 * backward). Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
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
 * to the directions the normalisation removes), special values.
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
