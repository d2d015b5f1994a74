/*
 * TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.
 *
 * Plain-C, single-threaded restatement of what the GPT-NeoX fused CUDA kernels
 * compute (scaled causal softmax, scaled padding-masked softmax, fused rotary
 * embedding; forward and backward). Only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load this library, and only as the checker.
 * Nothing under the product package imports, links or executes it.
 *
 * Each function cites the reference source it follows (paths relative to the
 * GPT-NeoX tree). Storage is fp16/bf16 (raw uint16_t bit patterns) or fp32;
 * all arithmetic is IEEE binary32, written so that no fused multiply-add is
 * formed (build with -ffp-contract=off), rounding to storage is to nearest even.
 *
 * Two documented choices where the reference leaves freedom or is inconsistent:
 *   - row sums are accumulated pairwise in fp32 (the reference sums per lane and
 *     then butterflies across the warp; any order is within a few fp32 ulp);
 *   - the forward `scale` is applied as the fp32 value handed in. The CUDA
 *     dispatcher narrows it to the input dtype first
 *     (scaled_upper_triang_masked_softmax.h:368, scaled_masked_softmax.h:358);
 *     pass an already narrowed value to reproduce that.
 * One definition that is this build's own, for a variant the reference's kernels do not have:
 *   - the attention-dropout mask is the counter-based one of layer_semantics.c: which
 *     elements torch's generator would drop is PARITY UNPINNED by construction, everything
 *     else about oracle_causal_softmax_dropout_fwd/bwd is the composition of pinned parts.
 *
 * How this oracle is pinned (tests/test_oracle_*.py): closed forms (row 0 of a
 * causal softmax is [1,0,...], constant rows give 1/(q+1), fully masked rows
 * give 1/sk), invariants (rows sum to 1, shift invariance, gradient rows sum to
 * 0, rotations preserve pair norms and compose to the identity, backward is the
 * adjoint of forward), brute force in float64 on tiny inputs, and the torch
 * library routines the reference's own Python fallback is made of.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>

#include "storage_formats.h"

/* exported for the conversion tests */
uint16_t oracle_float_to_bf16(float f) { return float_to_bf16(f); }
uint16_t oracle_float_to_f16(float f) { return float_to_f16(f); }
float oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
float oracle_f16_to_float(uint16_t h) { return f16_to_float(h); }

/* ------------------------------------------------------------------------ */
/* softmax of one row of already scaled/filled logits z[0..n) (fp32)         */
/* scaled_upper_triang_masked_softmax.h:206-233, scaled_masked_softmax.h:198-218 */
/* ------------------------------------------------------------------------ */
static void softmax_row(float* z, int64_t n)
{
    float m = z[0];
    for (int64_t k = 1; k < n; ++k) m = (m > z[k]) ? m : z[k];
    for (int64_t k = 0; k < n; ++k) z[k] = expf(z[k] - m);
    const float sum = pairwise_sum(z, n);
    for (int64_t k = 0; k < n; ++k) z[k] = z[k] / sum;
}

/*
 * scaled_upper_triang_masked_softmax_warp_forward
 * (scaled_upper_triang_masked_softmax.h:143-260): for row q of each [s,s]
 * matrix, softmax over columns k <= q of x*scale, +0 for k > q.
 * x, y: [batches, s, s].
 *
 * Two generalisations that the callers of the kernel apply around it with
 * tensors, restated here by index:
 *   window >= 0: columns k < q - window are masked as well -- the boolean mask
 *     of megatron/utils.py:67-80 (tril, then triu with diagonal -window);
 *   slopes != NULL: the AliBi matrix of
 *     megatron/model/positional_embeddings.py:219-257 is added to the scores
 *     first, in the storage dtype: a = dt(-(q-k)) (*) dt(slope[head]),
 *     x' = x (+) a, head = batch index % heads (transformer.py:584-585 adds it
 *     to the [b, np, sq, sk] scores before scale_mask_softmax);
 *   bias != NULL: `attention_scores += rpe` (transformer.py:580-582), a
 *     [heads, s, s] tensor in the storage dtype added (rounded) before AliBi.
 *   key_lengths != NULL: int32 [batches / heads]; the keys k >= key_lengths[b]
 *     of batch entry b = matrix / heads are padding and masked like the keys
 *     above the diagonal (the mask `causal | (k >= len)` given to
 *     forward_torch_softmax, fused_softmax.py:184-199). A row that keeps no
 *     key at all is 1/s in every column, above the diagonal too: what that
 *     fallback's softmax over a row of equal fill values gives.
 */
int oracle_causal_softmax_ex_fwd(void* y, const void* x, float scale, int64_t batches, int64_t s,
                                 int64_t window, const float* slopes, const void* bias,
                                 const int32_t* key_lengths, int64_t heads, int dt)
{
    if (dt != DT_F16 && dt != DT_BF16) return -1;
    float* z = (float*)malloc(sizeof(float) * (size_t)(s > 0 ? s : 1));
    if (!z) return -2;
    for (int64_t a = 0; a < batches; ++a) {
        const float slope = slopes ? round_to(slopes[a % heads], dt) : 0.0f;
        for (int64_t q = 0; q < s; ++q) {
            const int64_t base = (a * s + q) * s;
            const int64_t lo = (window >= 0 && q > window) ? q - window : 0;
            int64_t hi = q + 1; /* keys [lo, hi) take part */
            if (key_lengths) {
                const int64_t len = key_lengths[a / heads] < 0 ? 0 : key_lengths[a / heads];
                if (len < hi) hi = len;
            }
            if (hi <= lo) {
                for (int64_t k = 0; k < s; ++k) store_elem(y, base + k, dt, 1.0f / (float)s);
                continue;
            }
            for (int64_t k = lo; k < hi; ++k) {
                float v = load_elem(x, base + k, dt);
                /* attention_scores += rpe (transformer.py:580-582): bias [heads, s, s] in the storage dtype */
                if (bias) v = add_t(v, load_elem(bias, ((a % heads) * s + q) * s + k, dt), dt);
                if (slopes) {
                    const float dist = round_to(-(float)(q - k), dt);
                    v = add_t(v, mul_t(dist, slope, dt), dt);
                }
                z[k - lo] = v * scale;
            }
            softmax_row(z, hi - lo);
            for (int64_t k = 0; k < lo; ++k) store_elem(y, base + k, dt, 0.0f);
            for (int64_t k = lo; k < hi; ++k) store_elem(y, base + k, dt, z[k - lo]);
            for (int64_t k = hi; k < s; ++k) store_elem(y, base + k, dt, 0.0f);
        }
    }
    free(z);
    return 0;
}

int oracle_causal_softmax_fwd(void* y, const void* x, float scale, int64_t batches, int64_t s, int dt)
{
    return oracle_causal_softmax_ex_fwd(y, x, scale, batches, s, -1, NULL, NULL, NULL, 1, dt);
}

/*
 * scaled_masked_softmax_warp_forward (scaled_masked_softmax.h:117-238):
 * z = (mask == 1) ? -10000 : x*scale. x, y: [b, np, sq, sk];
 * mask: [pad_batches, 1, sq, sk] bytes, pad_batches in {1, b} (:141-147).
 */
int oracle_masked_softmax_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b,
                              int64_t np, int64_t sq, int64_t sk, int64_t pad_batches, int dt)
{
    if (dt != DT_F16 && dt != DT_BF16) return -1;
    if (pad_batches != 1 && pad_batches != b) return -3;
    float* z = (float*)malloc(sizeof(float) * (size_t)(sk > 0 ? sk : 1));
    if (!z) return -2;
    for (int64_t bi = 0; bi < b; ++bi)
        for (int64_t h = 0; h < np; ++h)
            for (int64_t q = 0; q < sq; ++q) {
                const int64_t base = ((bi * np + h) * sq + q) * sk;
                const uint8_t* mrow = mask + ((pad_batches == 1 ? 0 : bi) * sq + q) * sk;
                for (int64_t k = 0; k < sk; ++k)
                    z[k] = (mrow[k] != 1) ? load_elem(x, base + k, dt) * scale : -10000.0f;
                softmax_row(z, sk);
                for (int64_t k = 0; k < sk; ++k) store_elem(y, base + k, dt, z[k]);
            }
    free(z);
    return 0;
}

/*
 * scaled_upper_triang_masked_softmax_warp_backward (.h:262-361) when
 * causal != 0, scaled_masked_softmax_warp_backward (scaled_masked_softmax.h:240-335)
 * otherwise: g = dy*y on the unmasked columns (0 elsewhere),
 * dx = scale * (g - y * sum(g)). rows x n elements; rows_per_matrix gives the
 * causal row index q = row % rows_per_matrix. dx may alias dy.
 */
int oracle_softmax_ex_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows, int64_t n,
                          int64_t rows_per_matrix, int causal, int64_t window, const int32_t* key_lengths,
                          int64_t heads, int dt)
{
    if (dt != DT_F16 && dt != DT_BF16) return -1;
    float* g = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    float* p = (float*)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    if (!g || !p) {
        free(g);
        free(p);
        return -2;
    }
    for (int64_t r = 0; r < rows; ++r) {
        const int64_t q = r % rows_per_matrix;
        int64_t valid = causal ? q + 1 : n;
        if (causal && key_lengths) { /* padding keys, as in the forward */
            const int64_t len = key_lengths[(r / rows_per_matrix) / heads];
            if (len < valid) valid = len < 0 ? 0 : len;
        }
        /* sliding window: columns below q - window are masked like those above the diagonal */
        const int64_t lo = (causal && window >= 0 && q > window) ? q - window : 0;
        const int64_t base = r * n;
        for (int64_t k = 0; k < n; ++k) {
            if (k >= lo && k < valid) {
                p[k] = load_elem(y, base + k, dt);
                g[k] = load_elem(dy, base + k, dt) * p[k];
            } else {
                p[k] = 0.0f;
                g[k] = 0.0f;
            }
        }
        const float sum = pairwise_sum(g, n);
        for (int64_t k = 0; k < n; ++k) {
            const float t = p[k] * sum;
            const float d = g[k] - t;
            store_elem(dx, base + k, dt, scale * d);
        }
    }
    free(g);
    free(p);
    return 0;
}

/*
 * Causal softmax followed by attention dropout, as the attention layer applies them
 * (megatron/model/transformer.py:588-593: attention_probs = scale_mask_softmax(...), then
 * attention_probs = attention_dropout(attention_probs)): y as above, and
 * dropped = keep ? y_stored / (1 - p) : 0 computed from the stored (rounded) y and rounded again,
 * which is what a separate dropout kernel reading y produces. The mask is oracle_dropout_mask
 * (layer_semantics.c) over the flat element index of the [batches, s, s] tensor.
 */
int oracle_dropout_mask(uint8_t* keep, int64_t n, float p, uint64_t seed, uint64_t offset);

int oracle_causal_softmax_dropout_fwd(void* dropped, void* y, const void* x, float scale, int64_t batches, int64_t s,
                                      int64_t window, float p, uint64_t seed, uint64_t offset, int dt)
{
    int rc = oracle_causal_softmax_ex_fwd(y, x, scale, batches, s, window, NULL, NULL, NULL, 1, dt);
    if (rc) return rc;
    const int64_t n = batches * s * s;
    uint8_t* keep = (uint8_t*)malloc((size_t)(n > 0 ? n : 1));
    if (!keep) return -2;
    oracle_dropout_mask(keep, n, p, seed, offset);
    const float ds = (float)(1.0 / (1.0 - (double)p));
    for (int64_t e = 0; e < n; ++e) store_elem(dropped, e, dt, keep[e] ? load_elem(y, e, dt) * ds : 0.0f);
    free(keep);
    return 0;
}

/* Backward of the pair: first the dropout backward, g = keep ? dy / (1 - p) : 0 stored in the
 * storage type, then the softmax backward on g. dx may alias dy. */
int oracle_causal_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale, int64_t batches, int64_t s,
                                      int64_t window, float p, uint64_t seed, uint64_t offset, int dt)
{
    if (dt != DT_F16 && dt != DT_BF16) return -1;
    const int64_t n = batches * s * s;
    uint8_t* keep = (uint8_t*)malloc((size_t)(n > 0 ? n : 1));
    uint16_t* g = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)(n > 0 ? n : 1));
    if (!keep || !g) {
        free(keep);
        free(g);
        return -2;
    }
    oracle_dropout_mask(keep, n, p, seed, offset);
    const float ds = (float)(1.0 / (1.0 - (double)p));
    for (int64_t e = 0; e < n; ++e) store_elem(g, e, dt, keep[e] ? load_elem(dy, e, dt) * ds : 0.0f);
    int rc = oracle_softmax_ex_bwd(dx, g, y, scale, batches * s, s, s, 1, window, NULL, 1, dt);
    free(keep);
    free(g);
    return rc;
}

int oracle_softmax_bwd(void* dx, const void* dy, const void* y, float scale, int64_t rows, int64_t n,
                       int64_t rows_per_matrix, int causal, int dt)
{
    return oracle_softmax_ex_bwd(dx, dy, y, scale, rows, n, rows_per_matrix, causal, -1, NULL, 1, dt);
}

/*
 * get_batch_per_block (scaled_masked_softmax.h:338-352) for a machine whose
 * warp is `warp` lanes wide (32 on NVIDIA, 64 on gfx9).
 */
int oracle_batch_per_block(int64_t key_seq_len, int warp)
{
    int64_t pow2 = 1;
    while (pow2 < key_seq_len) pow2 *= 2;
    const int64_t ws = pow2 < warp ? pow2 : warp;
    const int64_t per_warp = pow2 <= 128 ? 2 : 1;
    return (int)((128 / ws) * per_warp);
}

/* ------------------------------------------------------------------------ */
/* rotary embedding                                                          */
/* ------------------------------------------------------------------------ */


/*
 * Shared body of the four rotary kernels
 * (fused_rotary_positional_embedding.h:27-74 fwd, :76-124 bwd, :126-174 cached
 * fwd, :176-225 cached bwd).
 *   cs_mode 0: cos/sin tables of dtype cs_dt, contiguous [s, d2]
 *   cs_mode 1: freqs fp32 [s, d2] in `cos`; cosf/sinf evaluated here
 * in/out: [s, b, h, d] with element strides is[4] / os[4].
 */
static int rope_any(void* out, const void* in, const void* cos, const void* sin, int64_t s, int64_t b,
                    int64_t h, int64_t d, int64_t d2, const int64_t* is, const int64_t* os, int dt,
                    int cs_dt, int cs_mode, int backward)
{
    if (dt != DT_F16 && dt != DT_BF16 && dt != DT_F32) return -1;
    if (d2 > d) return -3;
    const int64_t h2 = d2 / 2;
    for (int64_t si = 0; si < s; ++si)
        for (int64_t bi = 0; bi < b; ++bi)
            for (int64_t hi = 0; hi < h; ++hi) {
                const int64_t src = si * is[0] + bi * is[1] + hi * is[2];
                const int64_t dst = si * os[0] + bi * os[1] + hi * os[2];
                for (int64_t i = 0; i < d2; ++i) {
                    const int first = (i + h2 < d2);
                    const int64_t partner = first ? i + h2 : i + h2 - d2;
                    /* the index whose sine is used: own index forward, partner's backward */
                    const int64_t si_idx = backward ? partner : i;
                    float c, sn;
                    if (cs_mode == 0) {
                        c = round_to(load_elem(cos, si * d2 + i, cs_dt), dt);
                        sn = round_to(load_elem(sin, si * d2 + si_idx, cs_dt), dt);
                    } else {
                        c = round_to(cosf(((const float*)cos)[si * d2 + i]), dt);
                        sn = round_to(sinf(((const float*)cos)[si * d2 + si_idx]), dt);
                    }
                    const float x = load_elem(in, src + i * is[3], dt);
                    float r = load_elem(in, src + partner * is[3], dt);
                    if (!backward) {
                        if (first) r = -r; /* rotate_half: (-x2, x1) */
                    } else {
                        if (!first) sn = -sn;
                    }
                    const float v = add_t(mul_t(x, c, dt), mul_t(r, sn, dt), dt);
                    store_elem(out, dst + i * os[3], dt, v);
                }
                for (int64_t i = d2; i < d; ++i)
                    store_elem(out, dst + i * os[3], dt, load_elem(in, src + i * is[3], dt));
            }
    return 0;
}

int oracle_rope_cached(void* out, const void* in, const void* cos, const void* sin, int64_t s, int64_t b,
                       int64_t h, int64_t d, int64_t d2, const int64_t* is, const int64_t* os, int dt,
                       int cs_dt, int backward)
{
    if (cs_dt != DT_F32 && cs_dt != dt) return -1;
    return rope_any(out, in, cos, sin, s, b, h, d, d2, is, os, dt, cs_dt, 0, backward);
}

int oracle_rope_freqs(void* out, const void* in, const float* freqs, int64_t s, int64_t b, int64_t h,
                      int64_t d, int64_t d2, const int64_t* is, const int64_t* os, int dt, int backward)
{
    return rope_any(out, in, freqs, freqs, s, b, h, d, d2, is, os, dt, DT_F32, 1, backward);
}
