"""The caller of the fused softmax: scores -> probabilities -> context.

What ``ParallelSelfAttention.attention`` does in GPT-NeoX
(megatron/model/transformer.py:526-625) with the pieces of its constructor that
set the scaling (:417-424, :499-511), as a module of its own without the model
parallel layers around it:

    scores  = baddbmm(q, k^T) * (1 / norm_factor)          library GEMM (rocBLAS / hipBLASLt)
    probs   = softmax(scores * coeff + masks and biases)     one kernel of libneox_hotpath.so
    probs   = dropout(probs)                                 same kernel on the causal branch
    context = bmm(probs, v)                                  library GEMM

``norm_factor = sqrt(head_dim) * coeff`` and ``coeff = max(1, layer_number)`` with
``apply_query_key_layer_scaling``, otherwise ``coeff`` is None and the softmax does not
scale: the two factors cancel in exact arithmetic and only keep fp16 scores in range.

Everything between the two GEMMs that the reference runs as separate passes over
``[b, np, sq, sk]`` -- the relative-position bias add (:580-582), the AliBi add (:584-585),
the dropout (:592-593) -- is handed to ``FusedScaleMaskSoftmax`` and happens inside its
kernel. Tensors are laid out as in the reference: q ``[sq, b, np, hn]``, k and v
``[sk, b, np, hn]``, result ``[b, np, sq, hn]``.

Grouped-query attention (k and v with ``nkv < np`` heads): the reference repeats every k/v head
``np / nkv`` times before the rotary embedding and the GEMMs (``gqa_project``,
megatron/model/transformer.py:768-839). Here the heads are never repeated: the ``np / nkv`` query heads that
share a k/v head are stacked along the row dimension of the GEMMs (``[b * nkv, (np / nkv) * sq, hn]``), which
yields the same ``[b, np, sq, sk]`` scores, and the sum over the sharing heads in the gradients of k and v
happens inside the GEMM instead of in a reduction pass.
"""
import math

import torch

from .fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes
from .utils import get_fusion_type  # noqa: F401  (also reachable from here, where its caller lives)


class _ContextGemm(torch.autograd.Function):
    """``probs [B, sq, sk] x v [sk, B, hn] -> [sq, B, hn]``: the context GEMM writing the layout the output
    projection wants, which saves the ``permute(2, 0, 1, 3).contiguous()`` copy of
    megatron/model/transformer.py:941 and its counterpart in the backward (the library GEMM takes the
    strides; nothing is computed differently)."""

    @staticmethod
    def forward(ctx, probs, value):
        sk, batches, hn = value.shape
        out = torch.empty((probs.size(1), batches, hn), dtype=probs.dtype, device=probs.device)
        torch.bmm(probs, value.transpose(0, 1), out=out.transpose(0, 1))
        ctx.save_for_backward(probs, value)
        return out

    @staticmethod
    def backward(ctx, grad):
        probs, value = ctx.saved_tensors
        g = grad.transpose(0, 1)  # [B, sq, hn], a view
        grad_probs = torch.bmm(g, value.transpose(0, 1).transpose(1, 2)) if ctx.needs_input_grad[0] else None
        grad_value = torch.bmm(probs.transpose(1, 2), g).transpose(0, 1) if ctx.needs_input_grad[1] else None
        return grad_probs, grad_value


def causal_gemm_block(seq_len):
    """Rows per block of the blocked causal GEMMs, or 0 for one dense GEMM. Measured on the score, context and
    key-gradient GEMMs with 128 features per head: 512 at 2048 positions (-27 to -36 %), 1024 at 4096 and 8192
    (-17 to -40 %); at 1024 positions the smaller launches gain nothing."""
    if seq_len < 2048:
        return 0
    return 512 if seq_len < 4096 else 1024


def _row_blocks(seq_len, block, window):
    """``(r0, r1, c0)``: the queries ``[r0, r1)`` see the keys ``[c0, r1)`` -- ``c0`` is 0 without a sliding window
    and the start of the block that holds key ``r0 - window`` with one."""
    out = []
    for r0 in range(0, seq_len, block):
        c0 = 0 if window is None else max(0, (r0 - window) // block * block)
        out.append((r0, min(r0 + block, seq_len), c0))
    return out


def _column_blocks(seq_len, block, window):
    """``(c0, c1, r1)``: the keys ``[c0, c1)`` are seen by the queries ``[c0, r1)`` -- all later ones without a
    sliding window, those up to ``c1 - 1 + window`` with one."""
    out = []
    for c0 in range(0, seq_len, block):
        c1 = min(c0 + block, seq_len)
        out.append((c0, c1, seq_len if window is None else min(seq_len, c1 + window)))
    return out


class _CausalScoreGemm(torch.autograd.Function):
    """``alpha * q k^T`` for the causal softmax kernel, which never reads a score above the diagonal (or, with a
    sliding window, before the window): a block of rows is only computed for the keys its queries can see, the
    rest of the ``[B, s, s]`` result stays uninitialised. The gradient that comes back from the softmax backward
    is zero wherever the scores were not read, so the same blocks suffice for the gradients of q (row blocks) and
    k (column blocks). Same products as the dense GEMM on every element that is used; about ``(n + 1) / 2n`` of
    its work with ``n`` blocks and no window."""

    @staticmethod
    def forward(ctx, q, k, alpha, block, window):
        batches, s, _ = q.shape
        scores = torch.empty((batches, s, s), dtype=q.dtype, device=q.device)
        kt = k.transpose(1, 2)
        for r0, r1, c0 in _row_blocks(s, block, window):
            out = scores[:, r0:r1, c0:r1]
            if alpha == 1.0:
                torch.bmm(q[:, r0:r1], kt[:, :, c0:r1], out=out)
            else:
                torch.baddbmm(out, q[:, r0:r1], kt[:, :, c0:r1], beta=0.0, alpha=alpha, out=out)
        ctx.save_for_backward(q, k)
        ctx.conf = (alpha, block, window)
        return scores

    @staticmethod
    def backward(ctx, grad):
        q, k = ctx.saved_tensors
        alpha, block, window = ctx.conf
        batches, s, hn = q.shape
        grad_q = grad_k = None
        if ctx.needs_input_grad[0]:
            grad_q = torch.empty((batches, s, hn), dtype=q.dtype, device=q.device)
            for r0, r1, c0 in _row_blocks(s, block, window):
                torch.baddbmm(grad_q[:, r0:r1], grad[:, r0:r1, c0:r1], k[:, c0:r1], beta=0.0, alpha=alpha,
                              out=grad_q[:, r0:r1])
        if ctx.needs_input_grad[1]:
            grad_k = torch.empty((batches, s, hn), dtype=k.dtype, device=k.device)
            for c0, c1, r1 in _column_blocks(s, block, window):
                torch.baddbmm(grad_k[:, c0:c1], grad[:, c0:r1, c0:c1].transpose(1, 2), q[:, c0:r1], beta=0.0, alpha=alpha,
                              out=grad_k[:, c0:c1])
        return grad_q, grad_k, None, None, None


class _CausalContextGemm(torch.autograd.Function):
    """``probs v`` for probabilities that are zero above the diagonal and before the sliding window (the causal
    softmax kernel writes exact zeros there): a block of rows times the values its queries can see. The gradient
    of the probabilities is only computed on those blocks -- the softmax backward reads nothing else -- and the
    rest of that tensor stays uninitialised. ``merged``: write ``[sq, B, hn]`` (see ``_ContextGemm``) instead of
    ``[B, sq, hn]``."""

    @staticmethod
    def forward(ctx, probs, value, block, window, merged):
        batches, s, _ = probs.shape
        hv = value.size(2)
        if merged:
            result = torch.empty((s, batches, hv), dtype=probs.dtype, device=probs.device)
            out = result.transpose(0, 1)
        else:
            result = out = torch.empty((batches, s, hv), dtype=probs.dtype, device=probs.device)
        for r0, r1, c0 in _row_blocks(s, block, window):
            torch.bmm(probs[:, r0:r1, c0:r1], value[:, c0:r1], out=out[:, r0:r1])
        ctx.save_for_backward(probs, value)
        ctx.conf = (block, window, merged)
        return result

    @staticmethod
    def backward(ctx, grad):
        probs, value = ctx.saved_tensors
        block, window, merged = ctx.conf
        batches, s, _ = probs.shape
        g = grad.transpose(0, 1) if merged else grad   # [B, sq, hn]
        grad_probs = grad_value = None
        if ctx.needs_input_grad[0]:
            grad_probs = torch.empty_like(probs)
            vt = value.transpose(1, 2)
            for r0, r1, c0 in _row_blocks(s, block, window):
                torch.bmm(g[:, r0:r1], vt[:, :, c0:r1], out=grad_probs[:, r0:r1, c0:r1])
        if ctx.needs_input_grad[1]:
            grad_value = torch.empty((batches, s, value.size(2)), dtype=value.dtype, device=value.device)
            for c0, c1, r1 in _column_blocks(s, block, window):
                torch.bmm(probs[:, c0:r1, c0:c1].transpose(1, 2), g[:, c0:r1], out=grad_value[:, c0:c1])
        return grad_probs, grad_value, None, None, None


class CoreAttention(torch.nn.Module):
    """Unfused ("global") attention on top of the fused softmax.

    Arguments:
        head_dim: features per head (``hidden_size_per_attention_head``).
        layer_number: 1-based layer index, used by ``apply_query_key_layer_scaling``.
        fp16, bf16: the precision flags of the model (both False: fp32, torch softmax).
        fusion_type: a ``SoftmaxFusionTypes`` member.
        mask_func: ``mask_func(scores, mask)`` for the softmax's torch branch.
        attention_softmax_in_fp32, apply_query_key_layer_scaling: as in the reference's arguments;
            layer scaling forces the fp32 softmax (transformer.py:350-352).
        use_mup: divide by ``head_dim`` instead of its square root (transformer.py:423-424).
        attention_dropout, sliding_window_width, alibi_slopes: handed to the softmax module.
        rpe: optional module ``rpe(sq, sk) -> [1, np, sq, sk]`` (relative position bias).
        use_cache: crop the mask to the current key length (inference with a KV cache).
        fold_scale: apply ``1 / norm_factor`` inside the softmax kernel (as part of its fp32 scale) instead of
            as the ``alpha`` of the score GEMM, whose backward pays for ``alpha`` with an extra pass over the
            gradients of q and k. None (default): fold unless the scores are fp16 (there the scaled GEMM is
            what keeps them in range, the reason the reference scales twice) or the softmax is not in fp32.
        causal_gemm_blocks: with the causal kernel and sequences of 2048 positions or more, compute the two GEMMs
            (and the four of the backward) only on and below the diagonal blocks. The skipped parts of the score
            and probability tensors and of their gradients stay uninitialised; switch this off for tools that
            inspect those tensors (e.g. autograd's anomaly detection would report the stale NaN patterns in them).
    """

    def __init__(self, head_dim, layer_number, fp16, bf16, fusion_type, mask_func, attention_softmax_in_fp32=False,
                 apply_query_key_layer_scaling=False, use_mup=False, attention_dropout=0.0,
                 sliding_window_width=None, alibi_slopes=None, rpe=None, use_cache=False, fold_scale=None,
                 causal_gemm_blocks=True):
        super().__init__()
        self.causal_gemm_blocks = causal_gemm_blocks
        self.layer_number = max(1, int(layer_number))
        if apply_query_key_layer_scaling:
            attention_softmax_in_fp32 = True
        coeff = None
        self.norm_factor = math.sqrt(head_dim)
        if apply_query_key_layer_scaling:
            coeff = max(1, self.layer_number)
            self.norm_factor *= coeff
        if use_mup:
            self.norm_factor = head_dim
        self.rpe = rpe
        self.use_cache = use_cache
        if fold_scale is None:
            fold_scale = not fp16 and attention_softmax_in_fp32
        assert not fold_scale or attention_softmax_in_fp32, "a folded scale needs the softmax in fp32"
        # additive terms (rpe bias, AliBi) are added to the scores before the softmax scales them, so the
        # factor can only move behind the GEMM when there are none
        self.fold_scale = bool(fold_scale) and rpe is None and alibi_slopes is None
        self.gemm_alpha = 1.0 if self.fold_scale else 1.0 / self.norm_factor
        softmax_scale = (coeff or 1.0) / self.norm_factor if self.fold_scale else coeff
        self.scale_mask_softmax = FusedScaleMaskSoftmax(
            input_in_fp16=fp16, input_in_bf16=bf16, fusion_type=fusion_type, mask_func=mask_func,
            softmax_in_fp32=attention_softmax_in_fp32, scale=softmax_scale, sliding_window_width=sliding_window_width,
            alibi_slopes=alibi_slopes, attention_dropout=attention_dropout)

    def forward(self, query_layer, key_layer, value_layer, attention_mask, key_lengths=None, merged_heads=False):
        """Returns the context as ``[b, np, sq, hn]`` (what ``ParallelSelfAttention.attention`` returns), or with
        ``merged_heads`` as ``[sq, b, np * hn]``, the layout its caller brings it into before the output
        projection, written by the context GEMM itself."""
        b, np_, sq, sk = query_layer.size(1), query_layer.size(2), query_layer.size(0), key_layer.size(0)
        hn = query_layer.size(3)
        if key_layer.size(2) != np_:
            return self._forward_grouped(query_layer, key_layer, value_layer, attention_mask, key_lengths, merged_heads)
        # [sq, b, np, hn] -> [sq, b * np, hn]
        q = query_layer.reshape(sq, b * np_, hn)
        k = key_layer.reshape(sk, b * np_, hn)
        block = self._causal_block(attention_mask, b, np_, sq, sk, query_layer)
        if block:
            # the causal kernel neither reads scores nor leaves probabilities above the diagonal: skip those blocks
            window = self.scale_mask_softmax.sliding_window_width
            window = None if window is None or window < 0 else int(window)
            scores = _CausalScoreGemm.apply(q.transpose(0, 1), k.transpose(0, 1), self.gemm_alpha, block, window)
            bias = self.rpe(sq, sk) if self.rpe is not None else None
            # ... and is told that nobody reads the other blocks of its results, which it then does not write
            zero_block = block if block & (block - 1) == 0 else 0
            probs = self.scale_mask_softmax._forward_block_limited(scores.view(b, np_, sq, sk), attention_mask, bias,
                                                                   key_lengths, zero_block)
            v = value_layer.reshape(sk, b * np_, value_layer.size(3)).transpose(0, 1)
            context = _CausalContextGemm.apply(probs.view(b * np_, sq, sk), v, block, window, merged_heads)
            if merged_heads:
                return context.view(sq, b, np_ * value_layer.size(3))
            return context.view(b, np_, sq, value_layer.size(3))
        if self.fold_scale:
            scores = torch.bmm(q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2)).view(b, np_, sq, sk)
        else:
            scores = torch.empty((b * np_, sq, sk), dtype=q.dtype, device=q.device)
            scores = torch.baddbmm(scores, q.transpose(0, 1), k.transpose(0, 1).transpose(1, 2), beta=0.0,
                                   alpha=self.gemm_alpha).view(b, np_, sq, sk)
        if self.use_cache and attention_mask is not None:
            with torch.no_grad():
                attention_mask = attention_mask[..., :sk, :sk]
        bias = self.rpe(sq, sk) if self.rpe is not None else None
        probs = self.scale_mask_softmax(scores, attention_mask, bias=bias, key_lengths=key_lengths)
        # [sk, b, np, hn] -> [sk, b * np, hn]; context [b * np, sq, hn]
        v = value_layer.reshape(sk, b * np_, value_layer.size(3))
        if merged_heads:
            return _ContextGemm.apply(probs.view(b * np_, sq, sk), v).view(sq, b, np_ * value_layer.size(3))
        context = torch.bmm(probs.view(b * np_, sq, sk), v.transpose(0, 1))
        return context.view(b, np_, sq, value_layer.size(3))

    def _causal_block(self, attention_mask, b, np_, sq, sk, like):
        """Block size for the blocked causal GEMMs, 0 when the scores do not go to the causal kernel (which is what
        guarantees that nothing above the diagonal is read or left non-zero) or are too small to gain."""
        softmax = self.scale_mask_softmax
        if not self.causal_gemm_blocks or sq != sk or not like.is_cuda:
            return 0   # (with cached keys sq != sk except for the first call, which is an ordinary causal pass)
        if not (softmax.upper_triang_mask_fusion and softmax.is_kernel_available(attention_mask, b, np_, sq, sk)):
            return 0
        return causal_gemm_block(sq)

    def _forward_grouped(self, query_layer, key_layer, value_layer, attention_mask, key_lengths, merged_heads):
        """k and v ``[sk, b, nkv, hn]`` with ``nkv`` dividing ``np``: query head ``h`` attends with k/v head
        ``h // (np / nkv)`` (the order ``torch.repeat_interleave(k, np / nkv, dim=2)`` produces)."""
        sq, b, np_, hn = query_layer.shape
        sk, nkv, hv = key_layer.size(0), key_layer.size(2), value_layer.size(3)
        assert np_ % nkv == 0 and value_layer.size(2) == nkv, "query heads must be a multiple of the key/value heads"
        group = np_ // nkv
        if self._causal_block(attention_mask, b, np_, sq, sk, query_layer):
            # long causal sequences: skipping the blocks above the diagonal saves more than the grouped GEMMs do
            # (measured at 8192 positions, 8 of 32 heads), and the blocked GEMMs want one key head per query head
            key_layer = torch.repeat_interleave(key_layer, group, dim=2)
            value_layer = torch.repeat_interleave(value_layer, group, dim=2)
            return self.forward(query_layer, key_layer, value_layer, attention_mask, key_lengths, merged_heads)
        # [sq, b, nkv, group, hn] -> [b * nkv, group * sq, hn]: no copy when q was written head-major
        q = query_layer.view(sq, b, nkv, group, hn).permute(1, 2, 3, 0, 4).reshape(b * nkv, group * sq, hn)
        k = key_layer.permute(1, 2, 0, 3).reshape(b * nkv, sk, hn)
        v = value_layer.permute(1, 2, 0, 3).reshape(b * nkv, sk, hv)
        if self.fold_scale:
            scores = torch.bmm(q, k.transpose(1, 2))
        else:
            scores = torch.empty((b * nkv, group * sq, sk), dtype=q.dtype, device=q.device)
            scores = torch.baddbmm(scores, q, k.transpose(1, 2), beta=0.0, alpha=self.gemm_alpha)
        scores = scores.view(b, np_, sq, sk)
        if self.use_cache and attention_mask is not None:
            with torch.no_grad():
                attention_mask = attention_mask[..., :sk, :sk]
        bias = self.rpe(sq, sk) if self.rpe is not None else None
        probs = self.scale_mask_softmax(scores, attention_mask, bias=bias, key_lengths=key_lengths)
        context = torch.bmm(probs.view(b * nkv, group * sq, sk), v).view(b, np_, sq, hv)
        if merged_heads:
            return context.permute(2, 0, 1, 3).reshape(sq, b, np_ * hv)
        return context


def apply_rotary_to_query_key(query_layer, key_layer, rotary_emb, rotary_ndims=None, rope_fusion=True, bf16=False,
                              layer_past=None, one_launch=True):
    """The rotary block of ``ParallelSelfAttention.forward`` (megatron/model/transformer.py:877-914).

    ``query_layer`` ``[sq, b, np, hn]`` and ``key_layer`` ``[sq, b, nkv, hn]`` (possibly views of one fused
    projection output); ``rotary_emb`` a ``RotaryEmbedding`` over ``rotary_ndims`` features (None: all
    ``hn``); ``layer_past`` the cached ``(keys, values)`` of earlier positions when decoding.

    ``one_launch=True`` (fused path only): a single kernel launch rotates q and k, copies the features
    beyond ``rotary_ndims`` and starts at the position after the cache, so the slices, the two launches and
    the two concatenations of the reference disappear -- and the cached positions are honoured, which the
    reference's fused branch does not do (it passes no offset). ``one_launch=False`` follows the reference
    statement by statement.
    """
    from .fused_rope import fused_apply_rotary_pos_emb_cached, fused_apply_rotary_pos_emb_qk_cached
    from .positional_embeddings import apply_rotary_pos_emb, apply_rotary_pos_emb_torch

    seq_len = key_layer.shape[0]
    offset = 0
    if layer_past is not None and layer_past.numel() > 0:
        offset = layer_past[0].shape[0]
        seq_len += offset
    cos, sin = rotary_emb(key_layer, seq_len=seq_len)
    if rope_fusion and one_launch:
        return fused_apply_rotary_pos_emb_qk_cached(query_layer, key_layer, cos, sin, offset=offset)

    if rotary_ndims is not None:
        query_rot, query_pass = query_layer[..., :rotary_ndims], query_layer[..., rotary_ndims:]
        key_rot, key_pass = key_layer[..., :rotary_ndims], key_layer[..., rotary_ndims:]
    else:
        query_rot, key_rot = query_layer, key_layer
    if rope_fusion:
        # as the reference: positions 0..sq-1 whatever the cache holds
        rows = slice(0, query_rot.shape[0])
        query_layer, key_layer = (fused_apply_rotary_pos_emb_cached(rot, cos[rows], sin[rows]) for rot in (query_rot, key_rot))
    else:
        eager = apply_rotary_pos_emb_torch if bf16 else apply_rotary_pos_emb
        query_layer, key_layer = eager(query_rot, key_rot, cos, sin, offset=offset)
    if rotary_ndims is not None:
        query_layer = torch.cat((query_layer, query_pass), dim=-1)
        key_layer = torch.cat((key_layer, key_pass), dim=-1)
    return query_layer, key_layer


class _SplitRotaryQKV(torch.autograd.Function):
    """``[sq, b, np, 3 * hn]`` -> rotated q, rotated k (new contiguous tensors) and v (a view).

    Forward: one rotary launch reads q and k straight from the projection output. Backward: the two rotary
    backward kernels write into their slices of one gradient buffer for the projection output and the
    gradient of v is copied into the third slice, which replaces the concatenation that undoes
    ``torch.split`` (a pass over all three tensors) by a copy of one."""

    @staticmethod
    def forward(ctx, mixed, cos, sin):
        import fused_rotary_positional_embedding as ext

        hn = mixed.size(-1) // 3
        ctx.save_for_backward(cos, sin)
        q_rot, k_rot = ext.forward_cached_qk(mixed[..., :hn], mixed[..., hn:2 * hn], cos, sin, False)
        return q_rot, k_rot, mixed[..., 2 * hn:]

    @staticmethod
    def backward(ctx, grad_q, grad_k, grad_v):
        import fused_rotary_positional_embedding as ext

        cos, sin = ctx.saved_tensors
        like = next(g for g in (grad_q, grad_k, grad_v) if g is not None)
        sq, b, np_, hn = like.shape
        grad = torch.empty((sq, b, np_, 3 * hn), dtype=like.dtype, device=like.device)
        gq, gk, gv = grad[..., :hn], grad[..., hn:2 * hn], grad[..., 2 * hn:]
        if grad_q is not None and grad_k is not None:
            ext.backward_cached_qk(grad_q, grad_k, cos, sin, False, out=(gq, gk))
        else:
            for dst, g in ((gq, grad_q), (gk, grad_k)):
                if g is None:
                    dst.zero_()
                else:
                    dst.copy_(ext.backward_cached(g, cos, sin, False))
        if grad_v is None:
            gv.zero_()
        else:
            gv.copy_(grad_v)
        return grad, None, None


class _SplitRotaryGQA(torch.autograd.Function):
    """``[sq, b, (np + 2 * nkv) * hn]`` (all query heads, then the key heads, then the value heads:
    the layout of ``gqa_project``, megatron/model/transformer.py:774-794) -> rotated q ``[sq, b, np, hn]``,
    rotated k ``[sq, b, nkv, hn]`` and v (a view). q and k are written head-major (storage ``[b, heads, sq, hn]``),
    the layout in which the grouped GEMMs of ``CoreAttention`` take them without a copy. The backward writes the
    three gradients into one buffer for the projection output."""

    @staticmethod
    def forward(ctx, mixed, cos, sin, np_, nkv):
        import fused_rotary_positional_embedding as ext

        sq, b, total = mixed.shape
        hn = total // (np_ + 2 * nkv)
        ctx.save_for_backward(cos, sin)
        ctx.heads = (np_, nkv, hn)
        q_in = mixed[..., :np_ * hn].view(sq, b, np_, hn)
        k_in = mixed[..., np_ * hn:(np_ + nkv) * hn].view(sq, b, nkv, hn)
        q_out = torch.empty((b, np_, sq, hn), dtype=mixed.dtype, device=mixed.device).permute(2, 0, 1, 3)
        k_out = torch.empty((b, nkv, sq, hn), dtype=mixed.dtype, device=mixed.device).permute(2, 0, 1, 3)
        ext.forward_cached_qk(q_in, k_in, cos, sin, False, out=(q_out, k_out))
        return q_out, k_out, mixed[..., (np_ + nkv) * hn:].view(sq, b, nkv, hn)

    @staticmethod
    def backward(ctx, grad_q, grad_k, grad_v):
        import fused_rotary_positional_embedding as ext

        cos, sin = ctx.saved_tensors
        np_, nkv, hn = ctx.heads
        like = next(g for g in (grad_q, grad_k, grad_v) if g is not None)
        sq, b = like.shape[:2]
        grad = torch.empty((sq, b, (np_ + 2 * nkv) * hn), dtype=like.dtype, device=like.device)
        gq = grad[..., :np_ * hn].view(sq, b, np_, hn)
        gk = grad[..., np_ * hn:(np_ + nkv) * hn].view(sq, b, nkv, hn)
        gv = grad[..., (np_ + nkv) * hn:].view(sq, b, nkv, hn)
        if grad_q is not None and grad_k is not None:
            ext.backward_cached_qk(grad_q, grad_k, cos, sin, False, out=(gq, gk))
        else:
            for dst, g in ((gq, grad_q), (gk, grad_k)):
                if g is None:
                    dst.zero_()
                else:
                    dst.copy_(ext.backward_cached(g, cos, sin, False))
        if grad_v is None:
            gv.zero_()
        else:
            gv.copy_(grad_v)
        return grad, None, None, None, None


def split_gqa_and_rotate(mixed_x_layer, rotary_emb, num_heads, num_kv_heads, layer_past=None):
    """``split_qkv_and_rotate`` for grouped-query attention: ``mixed_x_layer`` is ``[sq, b, (np + 2 * nkv) * hn]``
    as ``gqa_project`` lays it out (megatron/model/transformer.py:774-794); returns query ``[sq, b, np, hn]``,
    key and value ``[sq, b, nkv, hn]`` -- the key/value heads are not repeated, ``CoreAttention`` groups the
    query heads instead."""
    seq_len = mixed_x_layer.shape[0]
    offset = 0
    if layer_past is not None and layer_past.numel() > 0:
        offset = layer_past[0].shape[0]
    cos, sin = rotary_emb(mixed_x_layer, seq_len=seq_len + offset)
    rows = slice(offset, offset + seq_len)
    return _SplitRotaryGQA.apply(mixed_x_layer, cos[rows], sin[rows], num_heads, num_kv_heads)


def split_qkv_and_rotate(mixed_x_layer, rotary_emb, layer_past=None):
    """The split of the fused projection output and the rotary block of ``ParallelSelfAttention.forward``
    (megatron/model/transformer.py:852-914) as one differentiable step: ``mixed_x_layer`` is
    ``[sq, b, np, 3 * hn]``; returns ``(query, key, value)``, each ``[sq, b, np, hn]``, query and key rotated
    over the first ``rotary_emb.dim`` features starting at the position after the cached keys."""
    seq_len = mixed_x_layer.shape[0]
    offset = 0
    if layer_past is not None and layer_past.numel() > 0:
        offset = layer_past[0].shape[0]
    cos, sin = rotary_emb(mixed_x_layer, seq_len=seq_len + offset)
    rows = slice(offset, offset + seq_len)
    return _SplitRotaryQKV.apply(mixed_x_layer, cos[rows], sin[rows])
