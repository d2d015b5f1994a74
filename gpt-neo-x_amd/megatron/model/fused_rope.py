"""Fused rotary positional embedding (RoPE) on MI355X, behind the public surface
of GPT-NeoX's ``megatron/model/fused_rope.py``: ``FusedRoPEFunc`` (:18-56),
``fused_apply_rotary_pos_emb`` (:59-76), ``FusedRoPECachedFunc`` (:79-117) and
``fused_apply_rotary_pos_emb_cached`` (:120-141), plus a q+k variant that the
reference does not have.

Layout: tensors are ``[s, b, h, d]`` with arbitrary strides (the q/k views of a
fused QKV projection need no ``.contiguous()``); tables are ``[s, 1, 1, d2]``
with ``d2 <= d``; features ``d2..d`` pass through unchanged.
``transpose_output_memory=True`` stores the result as ``[b, s, h, d]`` (returned
as an ``[s, b, h, d]`` view) so that ``out.transpose(0, 1)`` is contiguous.
"""
from typing import Tuple, Union

import torch

_Grads = Tuple[Union[torch.Tensor, None], ...]


def _kernels():
    import fused_rotary_positional_embedding

    return fused_rotary_positional_embedding


class FusedRoPEFunc(torch.autograd.Function):
    """RoPE from fp32 rotation angles; cos and sin are evaluated inside the kernel."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False) -> torch.Tensor:
        ctx.transpose_output_memory = transpose_output_memory
        ctx.save_for_backward(freqs)
        return _kernels().forward(t, freqs, transpose_output_memory)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> _Grads:
        (freqs,) = ctx.saved_tensors
        return _kernels().backward(grad_output, freqs, ctx.transpose_output_memory), None, None


class FusedRoPECachedFunc(torch.autograd.Function):
    """RoPE from precomputed cos / sin tables (fp32 or the dtype of the input)."""

    @staticmethod
    def forward(ctx, t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor,
                transpose_output_memory: bool = False) -> torch.Tensor:
        ctx.transpose_output_memory = transpose_output_memory
        ctx.save_for_backward(cos_, sin_)
        return _kernels().forward_cached(t, cos_, sin_, transpose_output_memory)

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor) -> _Grads:
        cos_, sin_ = ctx.saved_tensors
        return _kernels().backward_cached(grad_output, cos_, sin_, ctx.transpose_output_memory), None, None, None


class FusedRoPEQKCachedFunc(torch.autograd.Function):
    """RoPE of q and k from precomputed tables in a single kernel launch."""

    @staticmethod
    def forward(ctx, q, k, cos_, sin_, transpose_output_memory=False):
        ctx.transpose_output_memory = transpose_output_memory
        ctx.save_for_backward(cos_, sin_)
        return _kernels().forward_cached_qk(q, k, cos_, sin_, transpose_output_memory)

    @staticmethod
    def backward(ctx, grad_q, grad_k):
        cos_, sin_ = ctx.saved_tensors
        gq, gk = _kernels().backward_cached_qk(grad_q, grad_k, cos_, sin_, ctx.transpose_output_memory)
        return gq, gk, None, None, None


class FusedRoPEQKFunc(torch.autograd.Function):
    """RoPE of q and k from float32 angles in a single kernel launch."""

    @staticmethod
    def forward(ctx, q, k, freqs, transpose_output_memory=False):
        ctx.transpose_output_memory = transpose_output_memory
        ctx.save_for_backward(freqs)
        return _kernels().forward_qk(q, k, freqs, transpose_output_memory)

    @staticmethod
    def backward(ctx, grad_q, grad_k):
        (freqs,) = ctx.saved_tensors
        gq, gk = _kernels().backward_qk(grad_q, grad_k, freqs, ctx.transpose_output_memory)
        return gq, gk, None, None


def fused_apply_rotary_pos_emb_qk(
    q: torch.Tensor, k: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``fused_apply_rotary_pos_emb`` for q ``[s, b, hq, d]`` and k ``[s, b, hk, d]`` in one launch."""
    return FusedRoPEQKFunc.apply(q, k, freqs, transpose_output_memory)


def fused_apply_rotary_pos_emb(
    t: torch.Tensor, freqs: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """Rotate ``t`` ``[s, b, h, d]`` by the float32 angles ``freqs`` ``[s, 1, 1, d2]``."""
    return FusedRoPEFunc.apply(t, freqs, transpose_output_memory)


def fused_apply_rotary_pos_emb_cached(
    t: torch.Tensor, cos_: torch.Tensor, sin_: torch.Tensor, transpose_output_memory: bool = False
) -> torch.Tensor:
    """Rotate ``t`` ``[s, b, h, d]`` with the cached tables ``cos_`` / ``sin_`` ``[s, 1, 1, d2]``
    (float32 or the dtype of ``t``)."""
    return FusedRoPECachedFunc.apply(t, cos_, sin_, transpose_output_memory)


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

    q is ``[s, b, hq, d]``, k is ``[s, b, hk, d]`` (any strides; hk may differ from
    hq). The tables are ``[S, 1, 1, d2]`` with ``S >= offset + s`` and ``d2 <= d``;
    features ``d2..d`` pass through, so a partial rotary needs neither slicing nor
    concatenation. ``offset`` is the position of the first row (decoding with a
    key/value cache). Returns ``(q_rotated, k_rotated)``.
    """
    rows = slice(offset, offset + q.shape[0])
    return FusedRoPEQKCachedFunc.apply(q, k, cos_[rows, ...], sin_[rows, ...], transpose_output_memory)
