/*
 * neox_hotpath.h -- C ABI of libneox_hotpath.so
 *
 * MI355X (gfx950) implementation of the three GPT-NeoX fused kernels:
 * scaled upper-triangular (causal) masked softmax, scaled padding-masked
 * softmax and fused rotary positional embedding, forward and backward.
 *
 * Conventions shared by every entry point
 *   - all tensor arguments are raw DEVICE pointers; the library never
 *     allocates, frees, retains or synchronises on them;
 *   - sizes and strides are int64_t, strides are counted in ELEMENTS;
 *   - `dtype` is an nhp_dtype value; `stream` is a hipStream_t passed as
 *     void* (NULL = the legacy default stream);
 *   - the call only enqueues work on `stream` and returns; the return value
 *     is NHP_OK (0) or a negative nhp_status; nothing is launched when an
 *     error is returned; no C++ exception crosses the boundary;
 *   - the library keeps no mutable global state and is safe to call from
 *     several host threads at once (forward from the main thread, backward
 *     from autograd worker threads).
 *
 * Each declaration cites the reference interface it replaces; paths are
 * relative to the GPT-NeoX source tree.
 */
#ifndef NEOX_HOTPATH_H
#define NEOX_HOTPATH_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum nhp_dtype {
    NHP_F16 = 0,  /* IEEE binary16 */
    NHP_BF16 = 1, /* bfloat16 */
    NHP_F32 = 2   /* IEEE binary32 (rotary only) */
} nhp_dtype;

typedef enum nhp_status {
    NHP_OK = 0,
    NHP_ERR_DTYPE = -1,     /* dtype not supported by this entry point */
    NHP_ERR_SHAPE = -2,     /* a size is negative / inconsistent / beyond the supported range */
    NHP_ERR_NULL = -3,      /* a required pointer is NULL while the tensor is not empty */
    NHP_ERR_PAD_BATCHES = -4, /* mask batch dimension is neither 1 nor b */
    NHP_ERR_LAUNCH = -5,    /* hipGetLastError() reported a launch failure */
    NHP_ERR_ALIAS = -6,     /* an output overlaps an input where that is not allowed */
    NHP_ERR_SCRATCH = -7    /* the input needs more scratch memory than the entry point's fixed buffer holds */
} nhp_status;

/* Library ABI version (bumped when a signature changes). */
int nhp_abi_version(void);

/* Static, human readable text for an nhp_status value. Never NULL. */
const char* nhp_status_string(int status);

/* Longest softmax row (sk) the register-resident kernels accept; longer rows
 * take a slower streaming kernel but are still supported. */
int64_t nhp_softmax_max_resident_row(void);

/* Launch geometry the softmax kernels use for rows of `row_len` elements, for profiling
 * records (a measured figure belongs to one kernel instantiation): lanes per row L, 16-byte
 * chunks per lane K, waves per row W. `kind`: 0 causal forward, 1 causal forward with AliBi
 * or a bias tensor, 2 causal backward, 3 padding-mask forward, 4 padding-mask backward.
 * Returns NHP_ERR_SHAPE when such rows take the scalar kernel. Kind 0 describes the general
 * forward kernel; rows of at most 512 elements in tensors of enough rows (rows * L >= 2^20) with
 * nothing but the causal mask or a window take a kernel with the same L and four rows per lane,
 * which this query does not tell apart (the query has no row count). */
int nhp_softmax_geometry(int64_t row_len, int kind, int* lanes, int* chunks, int* waves);

/* ------------------------------------------------------------------------
 * Scaled upper-triangular (causal) masked softmax
 * ---------------------------------------------------------------------- */

/*
 * y[a, q, k] = softmax_k( scale * x[a, q, k] ) over k <= q,  +0 for k > q.
 * x, y: contiguous [attn_batches, seq_len, seq_len], fp16 or bf16; fp32
 * accumulation; elements k > q of x are never read.
 * y may alias x exactly (in-place) but must not partially overlap it.
 *
 * Replaces scaled_upper_triang_masked_softmax_cuda.forward
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-39
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax_cuda.cu:33-59
 *   kernel megatron/fused_kernels/scaled_upper_triang_masked_softmax.h:143-260
 * The reference's seq_len <= 2048 limit does not apply.
 */
int nhp_causal_softmax_fwd(void* y, const void* x, float scale,
                           int64_t attn_batches, int64_t seq_len,
                           int dtype, void* stream);

/*
 * dx[a, q, k] = scale * ( dy*y - y * sum_{j<=q} dy[j]*y[j] ) for k <= q,
 * +0 for k > q.  dy, y, dx: contiguous [attn_batches, seq_len, seq_len].
 * dx may alias dy exactly (the reference always works in place on dy).
 *
 * Replaces scaled_upper_triang_masked_softmax_cuda.backward
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:41-56
 *   megatron/fused_kernels/scaled_upper_triang_masked_softmax_cuda.cu:61-90
 *   kernel megatron/fused_kernels/scaled_upper_triang_masked_softmax.h:262-361
 */
int nhp_causal_softmax_bwd(void* dx, const void* dy, const void* y, float scale,
                           int64_t attn_batches, int64_t seq_len,
                           int dtype, void* stream);

/*
 * Causal softmax with the generalisations its caller needs, so that no mask
 * tensor is read and no biased copy of the scores is written:
 *
 *  window >= 0: sliding-window attention. Row q attends to columns
 *      max(0, q - window) <= k <= q (the mask megatron/utils.py:67-80 builds
 *      with sliding_window_width = window); everything else is +0 and is never
 *      read. window < 0 (or >= seq_len): plain causal.
 *  alibi_slopes != NULL: AliBi. The score of head hd = a % heads (a = index
 *      along attn_batches, i.e. x is a [b, heads, s, s] tensor) becomes
 *      x (+) ( dt(-(q - k)) (*) dt(slopes[hd]) ), every operation rounded to
 *      the storage dtype, which is what `scores + alibi_matrix` computes in
 *      eager torch (megatron/model/positional_embeddings.py:129-257, applied
 *      at megatron/model/transformer.py:584-585) before the softmax sees the
 *      scores. slopes: `heads` fp32 values on the device.
 *  bias != NULL: an additive bias [heads, seq_len, seq_len] in the storage
 *      dtype, shared by the batch (the relative-position bias added at
 *      megatron/model/transformer.py:580-582 as `attention_scores += rpe`):
 *      the score becomes x (+) bias[hd, q, k], rounded to the storage dtype,
 *      before AliBi (if any) and the softmax. Only the attended band is read.
 *  key_lengths != NULL: `attn_batches / heads` int32 values on the device, one
 *      per batch entry (x is a [b, heads, s, s] tensor): the keys
 *      k >= key_lengths[b] are padding and masked like the keys above the
 *      diagonal, i.e. the mask `causal | (k >= len)` handed to
 *      FusedScaleMaskSoftmax.forward (megatron/model/fused_softmax.py:140-146),
 *      which the reference's causal kernel ignores. Padding keys are never
 *      read. A row left without any key (length 0, or a window that starts in
 *      the padding) is 1/seq_len in every column, as the softmax of the
 *      reference's torch branch over a row of equal fill values.
 *      Values below 0 count as 0, values above seq_len as seq_len.
 *
 * The backward takes the same window and key_lengths (masked positions get
 * +0, the row sum runs over the attended keys only); AliBi and the bias tensor
 * are additive constants and do not appear in it.
 *
 * Extends scaled_upper_triang_masked_softmax_cuda.forward / backward
 * (megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-56), whose
 * kernel ignores the mask contents and therefore drops a sliding window
 * (megatron/model/fused_softmax.py:148-179).
 */
int nhp_causal_softmax_ex_fwd(void* y, const void* x, float scale,
                              int64_t attn_batches, int64_t seq_len,
                              int64_t window, const float* alibi_slopes, const void* bias,
                              const int32_t* key_lengths, int64_t heads, int dtype, void* stream);

int nhp_causal_softmax_ex_bwd(void* dx, const void* dy, const void* y, float scale,
                              int64_t attn_batches, int64_t seq_len, int64_t window,
                              const int32_t* key_lengths, int64_t heads, int dtype, void* stream);

/*
 * Causal softmax and attention dropout in one pass:
 *   y       = the probabilities of nhp_causal_softmax_ex_fwd (window as there; needed by the backward),
 *   dropped = keep ? y / (1 - p) : 0, formed from the stored y and rounded to the storage type,
 * i.e. what attention_probs = attention_dropout(scale_mask_softmax(...)) leaves in memory
 * (megatron/model/transformer.py:588-593), without the pass that re-reads y and without a stored mask.
 * The keep mask is the counter-based one of nhp_bias_dropout_add over the flat element index of the
 * [attn_batches, seq_len, seq_len] tensor, regenerated by the backward from (seed, offset):
 *   dx = softmax backward of g = keep ? dy / (1 - p) : 0 (g rounded to the storage type).
 * dx may alias dy; dropped must not alias y or x. Which elements are dropped differs from what
 * torch's generator would pick (see nhp_bias_dropout_add).
 *
 * Replaces scaled_upper_triang_masked_softmax_cuda.forward / backward
 * (megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-56) followed / preceded by
 * torch.nn.Dropout (self.attention_dropout, megatron/model/transformer.py:509,592-593).
 */
int nhp_causal_softmax_dropout_fwd(void* dropped, void* y, const void* x, float scale,
                                   int64_t attn_batches, int64_t seq_len, int64_t window,
                                   float p, uint64_t seed, uint64_t offset, int dtype, void* stream);

int nhp_causal_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale,
                                   int64_t attn_batches, int64_t seq_len, int64_t window,
                                   float p, uint64_t seed, uint64_t offset, int dtype, void* stream);

/*
 * The causal softmax entry points above for a caller that consumes the [seq_len, seq_len] matrices in
 * square blocks of `zero_block` rows and columns and skips the blocks that hold no visible (query, key)
 * pair -- the batched GEMMs either side of the softmax in ParallelSelfAttention.attention
 * (megatron/model/transformer.py:556-621: baddbmm before, bmm after) computed block by block. Row q of
 * y / dropped / dx is written from the start of the block that holds the first key visible to the first
 * row of q's block (column 0 without a window) to the end of the block that holds the diagonal, zeros
 * included; the columns outside that range are neither read nor written. zero_block: a power of two >= 8, or 0 for the whole row
 * (then these are exactly nhp_causal_softmax_ex_* / nhp_causal_softmax_dropout_*). Rows that take the
 * scalar kernels (seq_len not a multiple of 8, unaligned pointers) are written whole.
 * Replaces scaled_upper_triang_masked_softmax_cuda.forward / backward
 * (megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-56), whose zeros above the diagonal
 * are a third of the forward's memory traffic.
 */
int nhp_causal_softmax_blocks_fwd(void* y, const void* x, float scale, int64_t attn_batches,
                                  int64_t seq_len, int64_t window, int64_t zero_block,
                                  const float* alibi_slopes, const void* bias,
                                  const int32_t* key_lengths, int64_t heads, int dtype, void* stream);

int nhp_causal_softmax_blocks_bwd(void* dx, const void* dy, const void* y, float scale,
                                  int64_t attn_batches, int64_t seq_len, int64_t window,
                                  int64_t zero_block, const int32_t* key_lengths, int64_t heads,
                                  int dtype, void* stream);

int nhp_causal_softmax_dropout_blocks_fwd(void* dropped, void* y, const void* x, float scale,
                                          int64_t attn_batches, int64_t seq_len, int64_t window,
                                          int64_t zero_block, float p, uint64_t seed, uint64_t offset,
                                          int dtype, void* stream);

int nhp_causal_softmax_dropout_blocks_bwd(void* dx, const void* dy, const void* y, float scale,
                                          int64_t attn_batches, int64_t seq_len, int64_t window,
                                          int64_t zero_block, float p, uint64_t seed, uint64_t offset,
                                          int dtype, void* stream);

/*
 * Attention dropout together with the per-head extras of nhp_causal_softmax_ex_fwd (AliBi slopes, additive
 * bias tensor, key lengths; any of them may be NULL) and the block-limited writing of
 * nhp_causal_softmax_blocks_fwd, in one kernel: the scores pass through bias, AliBi, scaling, the band
 * mask, the softmax and the dropout exactly as in the entry points that do one of these at a time. The
 * backward takes the gradient of `dropped`, with the key lengths of the forward.
 *
 * Replaces, in ParallelSelfAttention.attention (megatron/model/transformer.py:580-593), the sequence
 * `attention_scores += rpe`, `alibi_embed(attention_scores)`, scale_mask_softmax (the fused branch:
 * megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:31-56) and attention_dropout.
 */
int nhp_causal_softmax_ex_dropout_fwd(void* dropped, void* y, const void* x, float scale,
                                      int64_t attn_batches, int64_t seq_len, int64_t window,
                                      int64_t zero_block, const float* alibi_slopes, const void* bias,
                                      const int32_t* key_lengths, int64_t heads, float p, uint64_t seed,
                                      uint64_t offset, int dtype, void* stream);

int nhp_causal_softmax_ex_dropout_bwd(void* dx, const void* dy, const void* y, float scale,
                                      int64_t attn_batches, int64_t seq_len, int64_t window,
                                      int64_t zero_block, const int32_t* key_lengths, int64_t heads,
                                      float p, uint64_t seed, uint64_t offset, int dtype, void* stream);

/*
 * nhp_masked_softmax_fwd with what the caller of the reference does to the scores and the mask before
 * the padding-mask softmax (megatron/model/transformer.py:580-588), done inside the kernel instead of in
 * full passes over [b, np, sq, sk] (any of the three may be NULL):
 *   bias         [np, sq, sk] in the scores' dtype, shared by the batch (`attention_scores += rpe`): added
 *                in the storage dtype, as the eager in-place addition leaves it in memory;
 *   alibi_slopes [np] fp32, needs sq == sk: the AliBi bias -(q - k) * slope for k <= q and nothing above
 *                the diagonal, with the roundings of AliBi.forward
 *                (megatron/model/positional_embeddings.py:219-257), after the bias;
 *   key_lengths  [b] int32: keys k >= key_lengths[b] count as masked (as if their mask bytes were 1).
 * Results are those of nhp_masked_softmax_fwd on scores and a mask prepared that way (bit-identical with
 * key_lengths alone; with AliBi or a bias the kernel takes another launch shape, hence another summation
 * order: within 1 ulp, zeros in the same places). The
 * backward is nhp_masked_softmax_bwd (it takes no mask). The _dropout variant also writes
 * dropped = dropout(y) as nhp_masked_softmax_dropout_fwd does; its backward is
 * nhp_masked_softmax_dropout_bwd.
 *
 * Replaces scaled_masked_softmax_cuda.forward (megatron/fused_kernels/scaled_masked_softmax.cpp:33-42)
 * together with those preparations.
 */
int nhp_masked_softmax_ex_fwd(void* y, const void* x, const uint8_t* mask, float scale, int64_t b,
                              int64_t np, int64_t sq, int64_t sk, int64_t pad_batches,
                              const float* alibi_slopes, const void* bias, const int32_t* key_lengths,
                              int dtype, void* stream);

int nhp_masked_softmax_ex_dropout_fwd(void* dropped, void* y, const void* x, const uint8_t* mask,
                                      float scale, int64_t b, int64_t np, int64_t sq, int64_t sk,
                                      int64_t pad_batches, const float* alibi_slopes, const void* bias,
                                      const int32_t* key_lengths, float p, uint64_t seed,
                                      uint64_t offset, int dtype, void* stream);

/*
 * The same for the padding-mask softmax: y as nhp_masked_softmax_fwd, dropped = keep ? y / (1 - p) : 0
 * over the flat element index of the [b, np, sq, sk] tensor; the backward is nhp_masked_softmax_bwd of
 * g = keep ? dy / (1 - p) : 0 (rows = b * np * sq).
 *
 * Replaces scaled_masked_softmax_cuda.forward / backward
 * (megatron/fused_kernels/scaled_masked_softmax.cpp:33-59) followed / preceded by torch.nn.Dropout
 * (self.attention_dropout, megatron/model/transformer.py:509,592-593).
 */
int nhp_masked_softmax_dropout_fwd(void* dropped, void* y, const void* x, const uint8_t* mask,
                                   float scale, int64_t b, int64_t np, int64_t sq, int64_t sk,
                                   int64_t pad_batches, float p, uint64_t seed, uint64_t offset,
                                   int dtype, void* stream);

int nhp_masked_softmax_dropout_bwd(void* dx, const void* dy, const void* y, float scale,
                                   int64_t rows, int64_t sk, float p, uint64_t seed, uint64_t offset,
                                   int dtype, void* stream);

/* ------------------------------------------------------------------------
 * Scaled padding-masked softmax
 * ---------------------------------------------------------------------- */

/*
 * z = (mask == 1) ? -10000 : scale * x ;  y = softmax over the last dim.
 * x, y: contiguous [b, np, sq, sk], fp16 or bf16.
 * mask: contiguous [pad_batches, 1, sq, sk], one byte per element (bool or
 * uint8; only the value 1 masks), pad_batches is 1 (shared by all batches)
 * or b. A fully masked row yields the uniform distribution 1/sk.
 *
 * Replaces scaled_masked_softmax_cuda.forward
 *   megatron/fused_kernels/scaled_masked_softmax.cpp:33-42
 *   megatron/fused_kernels/scaled_masked_softmax_cuda.cu:38-76
 *   kernel megatron/fused_kernels/scaled_masked_softmax.h:117-238
 * The reference's sk <= 2048 limit does not apply.
 */
int nhp_masked_softmax_fwd(void* y, const void* x, const uint8_t* mask, float scale,
                           int64_t b, int64_t np, int64_t sq, int64_t sk,
                           int64_t pad_batches, int dtype, void* stream);

/*
 * dx = scale * ( dy*y - y * sum_k dy*y ) per row; no mask is applied.
 * dy, y, dx: contiguous, `rows` rows of `sk` elements (rows = b*np*sq).
 * dx may alias dy exactly.
 *
 * Replaces scaled_masked_softmax_cuda.backward
 *   megatron/fused_kernels/scaled_masked_softmax.cpp:44-59
 *   megatron/fused_kernels/scaled_masked_softmax_cuda.cu:78-108
 *   kernel megatron/fused_kernels/scaled_masked_softmax.h:240-335
 */
int nhp_masked_softmax_bwd(void* dx, const void* dy, const void* y, float scale,
                           int64_t rows, int64_t sk, int dtype, void* stream);

/*
 * Rows handled per 128-thread block by the reference's launch geometry on a
 * 64-wide wavefront; only used by FusedScaleMaskSoftmax.is_kernel_available.
 * Returns a value >= 1, or a negative nhp_status if key_seq_len < 1.
 *
 * Replaces scaled_masked_softmax_cuda.get_batch_per_block
 *   megatron/fused_kernels/scaled_masked_softmax.cpp:61-64
 *   megatron/fused_kernels/scaled_masked_softmax.h:338-352
 */
int nhp_softmax_batch_per_block(int64_t query_seq_len, int64_t key_seq_len,
                                int64_t batches, int64_t attn_heads);

/* ------------------------------------------------------------------------
 * Fused rotary positional embedding (rotate-half form), sbhd layout
 * ---------------------------------------------------------------------- */

/*
 * For i < d2, h2 = d2/2:
 *   forward : out_i = in_i (*) c_i (+) rot_i (*) s_i,
 *             rot_i = (i < d2-h2) ? -in[i+h2] : in[i+h2-d2]
 *   backward: out_i = in_i (*) c_i (+) in[partner] (*) s'_i,
 *             s'_i  = (i < d2-h2) ? s[i+h2] : -s[i+h2-d2]
 * where c = cos[s_idx, i], s = sin[s_idx, i] are first converted to the data
 * dtype and (*) / (+) round to the data dtype after every operation (the
 * arithmetic of the 16-bit scalar types in the reference and of eager torch).
 * For d2 <= i < d the element is copied.
 *
 * in : [s, b, h, d] with arbitrary element strides in_stride[4];
 * out: [s, b, h, d] with arbitrary element strides out_stride[4] (a
 *      contiguous sbhd or bshd buffer in the reference); must not overlap in;
 * cos, sin: contiguous [s, d2]; cs_dtype is NHP_F32 or equal to dtype.
 * dtype: NHP_F16, NHP_BF16 or NHP_F32.
 *
 * Replaces fused_rotary_positional_embedding.forward_cached / backward_cached
 *   megatron/fused_kernels/fused_rotary_positional_embedding.cpp:75-125
 *   megatron/fused_kernels/fused_rotary_positional_embedding_cuda.cu:218-335
 *   kernels megatron/fused_kernels/fused_rotary_positional_embedding.h:126-225
 */
int nhp_rope_cached_fwd(void* out, const void* in, const void* cos, const void* sin,
                        int64_t s, int64_t b, int64_t h, int64_t d, int64_t d2,
                        const int64_t in_stride[4], const int64_t out_stride[4],
                        int dtype, int cs_dtype, void* stream);

int nhp_rope_cached_bwd(void* out, const void* in, const void* cos, const void* sin,
                        int64_t s, int64_t b, int64_t h, int64_t d, int64_t d2,
                        const int64_t in_stride[4], const int64_t out_stride[4],
                        int dtype, int cs_dtype, void* stream);

/*
 * q and k of one attention layer rotated by one launch with the same tables:
 * exactly nhp_rope_cached_fwd / _bwd applied to (q_out, q_in) and (k_out, k_in).
 * q: [s, b, hq, d], k: [s, b, hk, d] (hk may differ from hq: grouped-query
 * attention), both with their own element strides. This is the fused form of
 * the reference's two-operand functions
 *   apply_rotary_pos_emb / apply_rotary_pos_emb_torch
 *   megatron/model/positional_embeddings.py:110-126
 * and of the call site megatron/model/transformer.py:877-914, which calls the
 * fused kernel once per tensor, slices [..., :d2] before and concatenates the
 * pass-through features after; with d2 < d the copy happens inside the
 * kernel. A position `offset` (KV-cache decoding, transformer.py:893-896) is
 * expressed by passing cos + offset*d2 and sin + offset*d2.
 * When q_in and k_in are the slices [..., 0:d] and [..., d:2d] of one fused
 * projection buffer (k_in == q_in + d elements, equal strides, hq == hk: how
 * transformer.py:852-866 produces them) and the outputs share their strides,
 * each row's q and k head vectors are read as one run; nothing else changes.
 */
int nhp_rope_cached_qk_fwd(void* q_out, void* k_out, const void* q_in, const void* k_in,
                           const void* cos, const void* sin,
                           int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                           const int64_t q_in_stride[4], const int64_t k_in_stride[4],
                           const int64_t q_out_stride[4], const int64_t k_out_stride[4],
                           int dtype, int cs_dtype, void* stream);

int nhp_rope_cached_qk_bwd(void* q_out, void* k_out, const void* q_in, const void* k_in,
                           const void* cos, const void* sin,
                           int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                           const int64_t q_in_stride[4], const int64_t k_in_stride[4],
                           const int64_t q_out_stride[4], const int64_t k_out_stride[4],
                           int dtype, int cs_dtype, void* stream);

/*
 * Same, with c = cosf(freqs[s_idx, i]) and s = sinf(freqs[s_idx, i]) evaluated
 * on the device in fp32 and then converted to the data dtype.
 * freqs: contiguous fp32 [s, d2].
 *
 * Replaces fused_rotary_positional_embedding.forward / backward
 *   megatron/fused_kernels/fused_rotary_positional_embedding.cpp:39-73
 *   megatron/fused_kernels/fused_rotary_positional_embedding_cuda.cu:24-137
 *   kernels megatron/fused_kernels/fused_rotary_positional_embedding.h:27-124
 */
int nhp_rope_freqs_fwd(void* out, const void* in, const float* freqs,
                       int64_t s, int64_t b, int64_t h, int64_t d, int64_t d2,
                       const int64_t in_stride[4], const int64_t out_stride[4],
                       int dtype, void* stream);

int nhp_rope_freqs_bwd(void* out, const void* in, const float* freqs,
                       int64_t s, int64_t b, int64_t h, int64_t d, int64_t d2,
                       const int64_t in_stride[4], const int64_t out_stride[4],
                       int dtype, void* stream);

/*
 * q and k in one launch from the angles, as nhp_rope_cached_qk_fwd / _bwd do from the tables:
 * exactly nhp_rope_freqs_fwd / _bwd applied to (q_out, q_in) and (k_out, k_in). Fused form of the
 * two calls of fused_apply_rotary_pos_emb (megatron/model/fused_rope.py:61-76) that a caller makes
 * for the query and the key of a layer (megatron/model/transformer.py:898-910 does so with the
 * cached variant).
 */
int nhp_rope_freqs_qk_fwd(void* q_out, void* k_out, const void* q_in, const void* k_in,
                          const float* freqs,
                          int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                          const int64_t q_in_stride[4], const int64_t k_in_stride[4],
                          const int64_t q_out_stride[4], const int64_t k_out_stride[4],
                          int dtype, void* stream);

int nhp_rope_freqs_qk_bwd(void* q_out, void* k_out, const void* q_in, const void* k_in,
                          const float* freqs,
                          int64_t s, int64_t b, int64_t hq, int64_t hk, int64_t d, int64_t d2,
                          const int64_t q_in_stride[4], const int64_t k_in_stride[4],
                          const int64_t q_out_stride[4], const int64_t k_out_stride[4],
                          int dtype, void* stream);

/* ------------------------------------------------------------------------
 * Element-wise neighbours of attention in the transformer layer
 *
 * The reference reaches these through TorchScript functions, not through an
 * extension module; the entry points below are what a binding for those
 * functions calls. Tensors are dense [rows, cols] (rows = all leading
 * dimensions flattened), the bias is [cols]. dtype: NHP_F16, NHP_BF16 or
 * NHP_F32, the same for every operand. Operands are widened to fp32, the
 * expression is evaluated in fp32 and rounded once to the storage type (what
 * a fused TorchScript kernel does; eager 16-bit torch rounds after every
 * operator). The tanh-GeLU is evaluated in an algebraically equal form without
 * tanh (see pointwise.hip); results agree with the written formula to 2
 * representable values or the fp32 noise of `1 + tanh`. Outputs may alias inputs.
 * ---------------------------------------------------------------------- */

/*
 * out = x * 0.5 * (1 + tanh(0.79788456 * x * (1 + 0.044715 * x * x))), x = bias + y.
 * bias may be NULL.
 *
 * Replaces bias_gelu
 *   megatron/model/activations.py:79-82 (called from GeLUFunction.forward :101-105,
 *   used by ParallelMLP, megatron/model/transformer.py:176-186)
 */
int nhp_bias_gelu_fwd(void* out, const void* y, const void* bias,
                      int64_t rows, int64_t cols, int dtype, void* stream);

/*
 * dx = ff * g with x = bias + y, t = tanh(0.79788456 * x * (1 + 0.044715 * x * x)),
 * ff = 0.5 * x * ((1 - t*t) * (0.79788456 + 0.1070322243 * x * x)) + 0.5 * (1 + t).
 *
 * dbias (optional, [cols] in `dtype`): the column sums of the stored dx,
 * accumulated in fp32 -- the reduction autograd performs on the second tensor
 * GeLUFunction.backward returns. It needs `workspace`, a device buffer of
 * nhp_bias_gelu_bwd_workspace_bytes(rows, cols, dtype) bytes, 16-byte aligned,
 * owned by the caller (0 bytes: none needed, NULL is accepted). The sums are
 * formed in a fixed order: results are reproducible from run to run.
 *
 * Replaces bias_gelu_back
 *   megatron/model/activations.py:88-97 (GeLUFunction.backward :107-112)
 */
int nhp_bias_gelu_bwd(void* dx, const void* g, const void* y, const void* bias,
                      void* dbias, void* workspace,
                      int64_t rows, int64_t cols, int dtype, void* stream);

int64_t nhp_bias_gelu_bwd_workspace_bytes(int64_t rows, int64_t cols, int dtype);

/*
 * out[c] = sum over rows of x[r, c], accumulated in fp32 in a fixed order
 * (reproducible from run to run) and rounded once: the reduction autograd
 * performs for a bias that was expanded over the rows, i.e. the bias gradient
 * of bias_dropout_add at the reference's call sites
 * (megatron/model/transformer.py:1229, 1271: bias.expand_as(residual);
 * megatron/model/fused_bias_dropout.py:28-35). `workspace`: fp32 partial rows,
 * nhp_column_sum_workspace_bytes() bytes (a few MiB, bounded whatever the
 * row count; 0 for shapes that take the scalar path).
 */
int nhp_column_sum(void* out, const void* x, void* workspace, int64_t rows, int64_t cols,
                   int dtype, void* stream);
int64_t nhp_column_sum_workspace_bytes(int64_t rows, int64_t cols, int dtype);

/*
 * out = residual + (x + bias): bias_dropout_add with dropout switched off
 * (training False or prob 0, when torch's dropout is the identity).
 * bias and residual may each be NULL.
 *
 * Replaces bias_dropout_add / bias_dropout_add_fused_inference (and
 * bias_dropout_add_fused_train with prob = 0)
 *   megatron/model/fused_bias_dropout.py:28-60
 *   (call sites megatron/model/transformer.py:1168-1178,1229-1246,1269-1320)
 */
int nhp_bias_add_residual(void* out, const void* x, const void* bias, const void* residual,
                          int64_t rows, int64_t cols, int dtype, void* stream);

/*
 * out = residual + ((x1 + bias1) + (x2 + bias2)), rounded where three nhp_bias_add_residual calls round
 * (t1 = round(x1 + bias1), t3 = round(t1 + (x2 + bias2)), out = round(residual + t3)):
 * the three element-wise passes with which the parallel-residual layer combines its two branches
 *   attention_output = bias_dropout_fn(attention_output, attention_bias, residual=None)
 *   output           = bias_dropout_fn(mlp_output, mlp_bias, residual=attention_output)
 *   output           = residual + output
 * (ParallelTransformerLayer.forward with gpt_j_residual, megatron/model/transformer.py:1229-1250,
 * on bias_dropout_add, megatron/model/fused_bias_dropout.py:28-60) in one, with dropout off; the result
 * is bit for bit that of three nhp_bias_add_residual calls. bias1 and bias2 may each be NULL (without
 * bias1 there is no first rounding); out may alias x1, x2 or residual.
 */
int nhp_bias_add_residual_pair(void* out, const void* x1, const void* bias1, const void* x2,
                               const void* bias2, const void* residual, int64_t rows, int64_t cols,
                               int dtype, void* stream);

/*
 * bias_dropout_add with dropout active (training and 0 < p < 1):
 *   out = residual + keep * (x + bias) / (1 - p),  dx = keep * g / (1 - p)
 * evaluated in fp32 and rounded once. The keep mask is not stored: element e
 * (flat index) is kept when 16 bits of Philox4x32-10(counter = (e / 8, offset),
 * key = seed) -- bits 16 * (e % 8) of the 128-bit output -- are below
 * round((1 - p) * 65536); forward and backward regenerate it from (seed, offset).
 * The generator is this library's own: which elements are dropped differs
 * from what torch's generator would drop for the same seed, the distribution
 * (independent Bernoulli(1 - p) per element) is the same. bias and residual
 * may be NULL; p = 0 keeps everything.
 *
 * Replaces bias_dropout_add / bias_dropout_add_fused_train
 *   megatron/model/fused_bias_dropout.py:28-50 (torch.nn.functional.dropout, differentiated by autograd)
 */
int nhp_bias_dropout_add(void* out, const void* x, const void* bias, const void* residual,
                         int64_t rows, int64_t cols, float p, uint64_t seed, uint64_t offset,
                         int dtype, void* stream);

int nhp_dropout_bwd(void* dx, const void* g, int64_t rows, int64_t cols,
                    float p, uint64_t seed, uint64_t offset, int dtype, void* stream);

/* Philox4x32-10 on the host, the generator of the dropout mask above (for known-answer tests);
 * megatron/model/fused_bias_dropout.py:31 is where the reference draws its mask. */
void nhp_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4]);

/*
 * Gated MLP activations. in: [rows, 2 * features]; the first `features` values
 * of a row are x, the last `features` the gates g (x, gate = in.chunk(2, dim=-1));
 * bias: [2 * features] or NULL, each half added to its half of the row.
 *   forward:  out[rows, features] = act(g) * x
 *   backward: din[rows, 2 * features] = (dy * act(g), dy * x * act'(g))
 * act (enum nhp_gate_act): swish g * sigmoid(g) (SwiGLU), exact erf GeLU
 * (GeGLU), relu (ReGLU), sigmoid (GLU), identity (bilinear). `out` / `din`
 * must not alias `in`.
 *
 * Replaces Gated_Activation.forward
 *   megatron/model/transformer.py:186-206 with the activations get_activation selects
 *   for geglu / reglu / bilinear / swiglu / glu, megatron/model/activations.py:30-49,
 *   swish :128-130 (the reference differentiates it with autograd).
 */
enum nhp_gate_act {
    NHP_GATE_SWISH = 0,
    NHP_GATE_GELU = 1,
    NHP_GATE_RELU = 2,
    NHP_GATE_SIGMOID = 3,
    NHP_GATE_IDENTITY = 4
};

int nhp_gated_act_fwd(void* out, const void* in, const void* bias,
                      int64_t rows, int64_t features, int act, int dtype, void* stream);

int nhp_gated_act_bwd(void* din, const void* dy, const void* in, const void* bias,
                      int64_t rows, int64_t features, int act, int dtype, void* stream);

/* ------------------------------------------------------------------------
 * LayerNorm and RMSNorm
 *
 * x, y, dy, dx: dense [rows, cols] in `dtype` (NHP_F16, NHP_BF16, NHP_F32);
 * every row is normalised over its `cols` elements. gamma / beta (scale /
 * offset) and their gradients: [cols] in `param_dtype`, which is `dtype` or
 * NHP_F32; each may be NULL. Statistics and arithmetic are fp32, results are
 * rounded once. mean / rstd / inv: fp32 [rows], written by the forward (NULL:
 * not wanted) and read by the backward.
 *
 * The backward needs `workspace` when a parameter gradient is asked for: a
 * 16-byte aligned device buffer of nhp_norm_bwd_workspace_bytes(rows, cols,
 * dtype) bytes owned by the caller (0: none needed). Parameter gradients are
 * summed in a fixed order: results are reproducible from run to run.
 * ---------------------------------------------------------------------- */

/*
 * y = ((x - mean) * rstd) * gamma + beta, mean and biased variance per row,
 * rstd = 1 / sqrt(var + eps).
 *
 * Replaces torch.nn.LayerNorm as handed out by get_norm
 *   megatron/model/norms.py:16,19-51 (norm = "layernorm"), used as input_layernorm,
 *   post_attention_layernorm and final norm, megatron/model/transformer.py:985-1040,1362
 * and the apex-backed MixedFusedLayerNorm, megatron/model/fused_layer_norm.py:34-153.
 */
int nhp_layernorm_fwd(void* y, float* mean, float* rstd, const void* x,
                      const void* gamma, const void* beta, float eps,
                      int64_t rows, int64_t cols, int dtype, int param_dtype, void* stream);

/*
 * xhat = (x - mean) * rstd, g = dy * gamma:
 *   dx = rstd * (g - (sum(g) + xhat * sum(g * xhat)) / cols)
 *   dgamma = column sums of dy * xhat, dbeta = column sums of dy (each optional).
 * The adjoint of nhp_layernorm_fwd, i.e. what autograd runs for torch.nn.LayerNorm
 *   (megatron/model/norms.py:16).
 */
int nhp_layernorm_bwd(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x,
                      const float* mean, const float* rstd, const void* gamma, void* workspace,
                      int64_t rows, int64_t cols, int dtype, int param_dtype, void* stream);

/*
 * nhp_layernorm_bwd without a workspace argument and without any allocation, for callers that
 * cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses
 * that forbid it). No counterpart in the reference. Same arguments and kernels as
 * nhp_layernorm_bwd; the partial sums of the parameter gradients go to a fixed device array of
 * NHP_NOALLOC_SCRATCH_BYTES bytes (16 MiB) that is part of the library image on
 * every GPU it runs on. The array holds 16 MiB / (8 * cols) pairs of fp32 partial rows. Where
 * nhp_layernorm_bwd would use more workgroups than that (at 16384 rows: more than 4096 columns), fewer
 * are launched and each covers more rows: dx is the same bit for bit, dgamma and dbeta are sums in
 * another order (equal within fp32 rounding of the sums, then rounded to the parameter dtype); where
 * it would not, every result is bit-identical to nhp_layernorm_bwd's. Rows of more than 262144
 * columns (fewer than 8 partial rows fit) return NHP_ERR_SCRATCH with parameter gradients (nothing
 * is launched); without parameter gradients any shape is accepted.
 * The caller's device must be current. All calls on one GPU share the array: calls that overlap
 * in time on one GPU (different streams or threads) race; calls on one stream are ordered.
 * Nothing needs clearing between calls (every partial row that is read was written by the
 * same call). The array's address is looked up on the first call on each device; make that
 * call outside a graph capture.
 */
#define NHP_NOALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
int nhp_layernorm_bwd_noalloc(void* dx, void* dgamma, void* dbeta, const void* dy, const void* x,
                              const float* mean, const float* rstd, const void* gamma, int64_t rows,
                              int64_t cols, int dtype, int param_dtype, void* stream);

/*
 * Two LayerNorms of one input in one pass each way: y1 = xhat * gamma1 + beta1, y2 = xhat * gamma2 + beta2
 * with shared mean / rstd, and in the backward one dx for both,
 *   g = dy1 * gamma1 + dy2 * gamma2,  dx = rstd * (g - (sum(g) + xhat * sum(g * xhat)) / cols)
 * (fp32, one rounding; autograd would round the two dx and add them), beside the parameter gradients of
 * both norms. The parallel-residual layer applies input_layernorm and post_attention_layernorm to the
 * same x (megatron/model/transformer.py:1195-1213, ParallelTransformerLayer.forward with gpt_j_residual).
 * `workspace`: nhp_layernorm_pair_bwd_workspace_bytes() bytes when any parameter gradient is wanted.
 * Rows of more than 16 KiB are accepted but run slower than two single calls would.
 */
int nhp_layernorm_pair_fwd(void* y1, void* y2, float* mean, float* rstd, const void* x,
                           const void* gamma1, const void* beta1, const void* gamma2,
                           const void* beta2, float eps, int64_t rows, int64_t cols, int dtype,
                           int param_dtype, void* stream);
int nhp_layernorm_pair_bwd(void* dx, void* dgamma1, void* dbeta1, void* dgamma2, void* dbeta2,
                           const void* dy1, const void* dy2, const void* x, const float* mean,
                           const float* rstd, const void* gamma1, const void* gamma2,
                           void* workspace, int64_t rows, int64_t cols, int dtype, int param_dtype,
                           void* stream);
int64_t nhp_layernorm_pair_bwd_workspace_bytes(int64_t rows, int64_t cols, int dtype);

/*
 * y = scale * (x * inv) + offset with
 *   eps_mode 1: inv = 1 / (||x||_2 * cols^(-1/2) + eps), the Python class
 *               RMSNorm.forward, megatron/model/norms.py:54-107 (p disabled);
 *   eps_mode 0: inv = 1 / sqrt(mean(x^2) + eps), the fused variants
 *               MixedFusedRMSNorm, megatron/model/fused_layer_norm.py:156-252;
 *   eps_mode 2: inv = 1 / max(||x||_2, eps), ScaleNorm.forward,
 *               megatron/model/norms.py:110-119 (its scalar g is passed as a
 *               `scale` vector of cols equal values).
 */
int nhp_rmsnorm_fwd(void* y, float* inv, const void* x, const void* scale, const void* offset,
                    float eps, int eps_mode,
                    int64_t rows, int64_t cols, int dtype, int param_dtype, void* stream);

/*
 * xhat = x * inv, g = dy * scale, s = sum(g * xhat):
 *   dx = inv * (g - xhat * s / (cols * rho)), rho = 1 (eps_mode 0) or 1 - eps * inv (eps_mode 1;
 *   rho <= 0, an all-zero row, drops the second term); eps_mode 2: dx = inv * (g - xhat * s)
 *   while ||x|| > eps (inv < 1 / eps), dx = inv * g for a clamped norm;
 *   dscale = column sums of dy * xhat, doffset = column sums of dy (each optional).
 * The adjoint of nhp_rmsnorm_fwd, i.e. what autograd runs for RMSNorm.forward
 *   (megatron/model/norms.py:85-107) and ScaleNorm.forward (:117-119).
 */
int nhp_rmsnorm_bwd(void* dx, void* dscale, void* doffset, const void* dy, const void* x,
                    const float* inv, const void* scale, void* workspace, float eps, int eps_mode,
                    int64_t rows, int64_t cols, int dtype, int param_dtype, void* stream);

/*
 * Partial RMSNorm (the `p` argument of RMSNorm, megatron/model/norms.py:87-94):
 * the statistic is taken over the first stat_cols columns of a row
 * (1 <= stat_cols <= cols; `cols` in the formulas above becomes stat_cols),
 * every column is scaled by it. In the backward the xhat * s term reaches
 * only the columns that took part in the statistic.
 */
int nhp_rmsnorm_partial_fwd(void* y, float* inv, const void* x, const void* scale,
                            const void* offset, float eps, int eps_mode, int64_t rows, int64_t cols,
                            int64_t stat_cols, int dtype, int param_dtype, void* stream);
int nhp_rmsnorm_partial_bwd(void* dx, void* dscale, void* doffset, const void* dy, const void* x,
                            const float* inv, const void* scale, void* workspace, float eps,
                            int eps_mode, int64_t rows, int64_t cols, int64_t stat_cols, int dtype,
                            int param_dtype, void* stream);

int64_t nhp_norm_bwd_workspace_bytes(int64_t rows, int64_t cols, int dtype);

#ifdef __cplusplus
}
#endif

#endif /* NEOX_HOTPATH_H */
