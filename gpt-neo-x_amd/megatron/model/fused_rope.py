"""Autograd wrappers of the fused rotary positional embedding, with the public
surface of GPT-NeoX's ``megatron/model/fused_rope.py`` (FusedRoPEFunc :18-56,
fused_apply_rotary_pos_emb :59-76, FusedRoPECachedFunc :79-117,
fused_apply_rotary_pos_emb_cached :120-141).

Tensors are in ``sbhd`` layout with arbitrary strides (no ``.contiguous()`` is
needed on the q/k views of a fused QKV projection); the rotary tables have
shape [s, 1, 1, d2] with d2 <= d, and features beyond d2 pass through.
"""
from typing import Tuple, Union

import torch


class FusedRoPEFunc(torch.autograd.Function):
    """RoPE from fp32 angles; cos/sin are evaluated inside the kernel."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False) -> torch.Tensor:
        import fused_rotary_positional_embedding as ext

        out = ext.forward(t, freqs, transpose_output_memory)
        ctx.save_for_backward(freqs)
        ctx.transpose_output_memory = transpose_output_memory
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> Tuple[Union[torch.Tensor, None], ...]:
        import fused_rotary_positional_embedding as ext

        (freqs,) = ctx.saved_tensors
        return ext.backward(grad_output, freqs, ctx.transpose_output_memory), None, None


def fused_apply_rotary_pos_emb(
    t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """Apply rotary positional embedding to ``t``.

    Args:
        t: [s, b, h, d] input.
        freqs: [s, 1, 1, d2] rotation angles, float32.
        transpose_output_memory: lay the result out as [b, s, h, d] in memory
            (returned as a [s, b, h, d] view), so that ``out.transpose(0, 1)``
            is contiguous.
    """
    return FusedRoPEFunc.apply(t, freqs, transpose_output_memory)


class FusedRoPECachedFunc(torch.autograd.Function):
    """RoPE from precomputed cos/sin tables."""

    @staticmethod
    def forward(
        ctx, t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor, transpose_output_memory: bool = False
    ) -> torch.Tensor:
        import fused_rotary_positional_embedding as ext

        out = ext.forward_cached(t, cos_, sin_, transpose_output_memory)
        ctx.save_for_backward(cos_, sin_)
        ctx.transpose_output_memory = transpose_output_memory
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> Tuple[Union[torch.Tensor, None], ...]:
        import fused_rotary_positional_embedding as ext

        cos_, sin_ = ctx.saved_tensors
        grad = ext.backward_cached(grad_output, cos_, sin_, ctx.transpose_output_memory)
        return grad, None, None, None


def fused_apply_rotary_pos_emb_cached(
    t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """Apply rotary positional embedding to ``t`` using cached tables.

    Args:
        t: [s, b, h, d] input.
        cos_, sin_: [s, 1, 1, d2] tables, float32 or the dtype of ``t``.
        transpose_output_memory: as in ``fused_apply_rotary_pos_emb``.
    """
    return FusedRoPECachedFunc.apply(t, cos_, sin_, transpose_output_memory)


class FusedRoPEQKCachedFunc(torch.autograd.Function):
    """RoPE of q and k from precomputed cos/sin tables in one kernel launch."""

    @staticmethod
    def forward(ctx, q, k, cos_, sin_, transpose_output_memory=False):
        import fused_rotary_positional_embedding as ext

        q_out, k_out = ext.forward_cached_qk(q, k, cos_, sin_, transpose_output_memory)
        ctx.save_for_backward(cos_, sin_)
        ctx.transpose_output_memory = transpose_output_memory
        return q_out, k_out

    @staticmethod
    def backward(ctx, grad_q, grad_k):
        import fused_rotary_positional_embedding as ext

        cos_, sin_ = ctx.saved_tensors
        gq, gk = ext.backward_cached_qk(grad_q, grad_k, cos_, sin_, ctx.transpose_output_memory)
        return gq, gk, None, None, None


def fused_apply_rotary_pos_emb_qk_cached(
    q: torch.Tensor,
    k: torch.Tensor,
    cos_: torch.Tensor,
    sin_: torch.Tensor,
    offset: int = 0,
    transpose_output_memory: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Fused counterpart of ``apply_rotary_pos_emb(q, k, cos, sin, offset)``
    (megatron/model/positional_embeddings.py:110-126): both tensors in one launch.

    Args:
        q: [s, b, hq, d]; k: [s, b, hk, d] (any strides; hk may differ from hq).
        cos_, sin_: [S, 1, 1, d2] tables with S >= offset + s and d2 <= d; features
            d2..d pass through, so a partial rotary needs no slicing and no concatenation.
        offset: position of the first row of q/k (decoding with a key/value cache).
        transpose_output_memory: as in ``fused_apply_rotary_pos_emb``.
    Returns (q_rotated, k_rotated).
    """
    s = q.shape[0]
    cos_ = cos_[offset : offset + s, ...]
    sin_ = sin_[offset : offset + s, ...]
    return FusedRoPEQKCachedFunc.apply(q, k, cos_, sin_, transpose_output_memory)
