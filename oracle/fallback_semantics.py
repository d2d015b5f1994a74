"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

Torch restatement of the reference's *Python* path for the hot ops, i.e. what
GPT-NeoX computes when the fused kernels are switched off. It is the CPU
baseline that bench.py times and a second, independent statement of the
semantics that the C oracle is cross-checked against.

Follows (paths relative to the GPT-NeoX tree):
  megatron/model/fused_softmax.py:184-199   forward_torch_softmax
  megatron/model/gpt2_model.py:49-57        gpt2_attention_mask_func
  megatron/utils.py:67-80                   get_attn_mask
  megatron/model/positional_embeddings.py:62-79   RotaryEmbedding._prepare_cache
  megatron/model/positional_embeddings.py:103-126 rotate_half / apply_rotary_pos_emb_torch
"""
import torch


def causal_mask(seq_len, device="cpu", sliding_window_width=None):
    """Boolean [1,1,s,s], True = masked: keys after the query, and with a sliding
    window also keys more than `sliding_window_width` before it
    (megatron/utils.py:67-80: tril, then triu(diagonal=-width), then `< 0.5`)."""
    idx = torch.arange(seq_len, device=device)
    masked = idx[None, :] > idx[:, None]
    if sliding_window_width is not None:
        masked = masked | (idx[None, :] < idx[:, None] - sliding_window_width)
    return masked.view(1, 1, seq_len, seq_len)


def alibi_slopes(n):
    """Per-head AliBi slopes (megatron/model/positional_embeddings.py:147-168)."""
    import math

    def power_of_2(m):
        start = 2 ** (-(2 ** -(math.log2(m) - 3)))
        return [start * start**i for i in range(m)]

    if math.log2(n).is_integer():
        return power_of_2(n)
    closest = 2 ** math.floor(math.log2(n))
    return power_of_2(closest) + alibi_slopes(2 * closest)[0::2][: n - closest]


def alibi_add(scores, slopes):
    """scores [b, np, s, s] + AliBi matrix, in scores.dtype, as AliBi.forward does for
    sq == sk (positional_embeddings.py:219-257): a = -tril(i - j), cast, times slopes."""
    s = scores.shape[-1]
    i = torch.arange(s, device=scores.device)
    a = -torch.tril(i.view(s, 1).repeat(1, s) + torch.arange(0, -s, -1, device=scores.device))
    a = a.to(scores.dtype)
    sl = slopes.to(a.device).to(a.dtype)
    a = a * sl.view(sl.shape[0], 1, 1)
    return scores + a


def fill_masked_with_dtype_min(scores, mask):
    """In-place fill of masked logits with the most negative finite value of
    their dtype (megatron/model/gpt2_model.py:49-57)."""
    scores.masked_fill_(mask, torch.finfo(scores.dtype).min)
    return scores


def torch_softmax_fallback(scores, mask, scale, softmax_in_fp32=True):
    """forward_torch_softmax (megatron/model/fused_softmax.py:184-199).

    scores [b, np, sq, sk] fp16/bf16, mask broadcastable bool (True = masked)
    or None, scale a float or None. Returns probabilities in scores.dtype.
    """
    half_in = scores.dtype in (torch.float16, torch.bfloat16)
    work = scores.float() if (half_in and softmax_in_fp32) else scores
    if scale is not None:
        work = work * scale
    if mask is not None:
        work = fill_masked_with_dtype_min(work, mask)
    probs = torch.softmax(work, dim=-1)
    if half_in and softmax_in_fp32:
        probs = probs.to(scores.dtype)
    return probs


def rotary_tables(dim, seq_len, base=10000, precision=torch.half):
    """cos/sin cache of RotaryEmbedding (positional_embeddings.py:62-79).

    Returns (cos, sin, angles): cos/sin [s,1,1,dim] in `precision`, angles
    [s,1,1,dim] fp32 (the `emb` attribute).
    """
    exponents = torch.arange(0, dim, 2).float() / dim
    inv_freq = 1.0 / (base**exponents)
    positions = torch.arange(seq_len).type_as(inv_freq)
    half = torch.outer(positions, inv_freq)
    angles = torch.cat((half, half), dim=-1)
    cos = angles.cos()[:, None, None, :].to(precision)
    sin = angles.sin()[:, None, None, :].to(precision)
    return cos, sin, angles.reshape(seq_len, 1, 1, dim)


def rotate_half(x):
    """(-x2, x1) with x split in halves along the last dim (positional_embeddings.py:103-107)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def eager_rotary(t, cos, sin, offset=0):
    """One operand of apply_rotary_pos_emb_torch (positional_embeddings.py:119-126):
    every product and the sum are rounded to t.dtype by torch."""
    cos = cos[offset : t.shape[0] + offset, ...]
    sin = sin[offset : t.shape[0] + offset, ...]
    return (t * cos) + (rotate_half(t) * sin)


def eager_rotary_partial(t, cos, sin):
    """Rotate the first cos.shape[-1] features and pass the rest through, the
    slice + cat sequence of ParallelSelfAttention (transformer.py:878-914)."""
    d2 = cos.shape[-1]
    if d2 == t.shape[-1]:
        return eager_rotary(t, cos, sin)
    return torch.cat((eager_rotary(t[..., :d2], cos, sin), t[..., d2:]), dim=-1)
