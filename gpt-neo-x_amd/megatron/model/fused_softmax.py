"""Scale + mask + softmax for attention scores on MI355X.

Public surface of GPT-NeoX's ``megatron/model/fused_softmax.py``:
``SoftmaxFusionTypes`` (:86-89), the autograd functions
``ScaledUpperTriangMaskedSoftmax`` (:24-53) and ``ScaledMaskedSoftmax`` (:56-83)
and the module ``FusedScaleMaskSoftmax`` (:92-205) with ``forward``,
``is_kernel_available``, ``forward_fused_softmax``, ``forward_torch_softmax``
and the static ``get_batch_per_block``.

The fused branches run hand-written gfx950 kernels, reached through the same
extension-module names the reference imports. What differs from the reference,
all of it widening:

* key lengths above 2048 stay on the fused branch (rows up to 65536 keys are
  held in registers, longer ones stream);
* ``scale`` reaches the forward kernel in fp32 by default, as on the reference's torch
  branch; the reference's CUDA dispatcher narrows it to the input dtype first, which the
  constructor argument ``narrow_forward_scale=True`` reproduces;
* two optional constructor arguments let the kernels do by index what their
  caller otherwise does with tensors: ``sliding_window_width`` (causal kernel; the
  reference's causal kernel never looks at the mask, so a sliding window is lost on
  its fused branch) and ``alibi_slopes`` (the AliBi bias is formed inside either
  kernel instead of by a separate ``scores + alibi_matrix`` pass). Both default to off;
* ``forward(input, mask, bias=None)``: an optional additive bias ``[1, np, sq, sk]``
  (the relative-position bias the caller adds with ``attention_scores += rpe``)
  is read by the kernel beside the scores instead of being added in a pass of its own;
* ``forward(..., key_lengths=None)``: an integer tensor ``[b]`` of real key counts for
  right-padded batches. Both kernels mask the padding keys by index (the reference's
  causal kernel ignores the mask, so padding is attended to on its fused branch); the
  torch branch merges ``k >= key_lengths[b]`` into the mask it is given;
* constructor argument ``attention_dropout`` (default 0): in training mode the module returns
  ``dropout(probabilities)``; on the fused branches softmax and dropout are one kernel, with or
  without the extras above, and the keep mask (the library's counter-based generator, seeded from
  the device's CUDA generator, see ``megatron.model.dropout_rng``) is regenerated in the backward instead of being stored. The caller must
  then not apply its own dropout.
"""
import enum

import torch
from torch import nn

from ..fused_kernels import load_fused_kernels
from . import dropout_rng


class SoftmaxFusionTypes(enum.Enum):
    upper_triang = 1  # causal mask
    general = 2  # general mask
    none = 3  # no fusion


def _scale_tensor(scale):
    # kept as a CPU fp32 tensor so that it can ride along in save_for_backward
    return torch.tensor([scale])


class ScaledUpperTriangMaskedSoftmax(torch.autograd.Function):
    """``softmax(scale * x)`` over the lower triangle of ``[attn_batches, sq, sk]``
    scores (zeros above the diagonal), one kernel forward and one backward.

    ``window``, ``alibi_slopes``, ``bias`` and ``key_lengths`` are the optional extras described in
    the module docstring; the reference signature is ``apply(inputs, scale)``.
    """

    @staticmethod
    def forward(ctx, inputs, scale, window=None, alibi_slopes=None, bias=None, key_lengths=None, zero_block=0,
                narrow_scale=False):
        import scaled_upper_triang_masked_softmax_cuda as kernels

        factor = _scale_tensor(scale)
        out = kernels.forward(inputs, factor[0], window, alibi_slopes, bias, key_lengths, zero_block,
                              narrow_scale=narrow_scale)
        ctx.window = window
        ctx.zero_block = zero_block
        ctx.bias_shape = None if bias is None else tuple(bias.shape)
        _save(ctx, out, factor, key_lengths)
        return out

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_upper_triang_masked_softmax_cuda as kernels

        out, factor, key_lengths = _saved(ctx)
        # in place on output_grads, like the reference kernel; the backward's factor is never narrowed
        # (scaled_upper_triang_masked_softmax.h:467 takes acc_t)
        grad = kernels.backward(output_grads, out, factor[0], ctx.window, key_lengths, ctx.zero_block)
        grad_bias = None
        if ctx.bias_shape is not None and ctx.needs_input_grad[4]:
            # the bias is shared by the batch: its gradient is the batch sum of the score gradient
            full = grad
            if ctx.zero_block:
                # the blocks the kernel did not write hold no gradient: leave them out of the sum
                sq = ctx.bias_shape[-2]
                full = torch.where(_written_blocks(sq, ctx.zero_block, ctx.window, grad.device), grad, torch.zeros_like(grad))
            grad_bias = _batch_sum(full, ctx.bias_shape)
        return grad, None, None, None, grad_bias, None, None, None


def _save(ctx, out, factor, key_lengths):
    """Keeps the tensors of a forward for its backward; the key lengths go through save_for_backward as well, so
    that autograd notices an in-place change between the two."""
    ctx.has_key_lengths = key_lengths is not None
    if ctx.has_key_lengths:
        ctx.save_for_backward(out, factor, key_lengths)
    else:
        ctx.save_for_backward(out, factor)


def _saved(ctx):
    if ctx.has_key_lengths:
        return ctx.saved_tensors
    return ctx.saved_tensors + (None,)


def _written_blocks(seq_len, zero_block, window, device):
    """[seq_len, seq_len] bool: the part of every row that the causal kernels write when called with ``zero_block``."""
    q = torch.arange(seq_len, device=device).view(seq_len, 1)
    k = torch.arange(seq_len, device=device).view(1, seq_len)
    hi = (q // zero_block + 1) * zero_block
    lo = torch.zeros_like(q)
    if window is not None and 0 <= window < seq_len:
        lo = (q // zero_block * zero_block - window).clamp(min=0) // zero_block * zero_block
    return (k < hi) & (k >= lo)


def _batch_sum(grad, bias_shape):
    """Gradient of a bias shared by the batch: the batch sum of the score gradient, in the bias's shape."""
    heads, sq, sk = bias_shape[-3:]
    return grad.view(-1, heads, sq, sk).sum(dim=0).view(bias_shape)


class ScaledUpperTriangMaskedSoftmaxDropout(torch.autograd.Function):
    """``dropout(softmax(scale * x))`` under the causal mask in one kernel forward and one backward, with the
    same optional extras as ``ScaledUpperTriangMaskedSoftmax``.
    No counterpart in the reference, which runs ``torch.nn.Dropout`` on the probabilities."""

    @staticmethod
    def forward(ctx, inputs, scale, prob, seed, window=None, zero_block=0, alibi_slopes=None, bias=None,
                key_lengths=None, narrow_scale=False):
        import scaled_upper_triang_masked_softmax_cuda as kernels

        factor = _scale_tensor(scale)
        dropped, probs = kernels.forward_dropout(inputs, factor[0], prob, seed, window, zero_block, alibi_slopes, bias,
                                                 key_lengths, narrow_scale=narrow_scale)
        ctx.conf = (float(prob), int(seed), window, zero_block)
        ctx.bias_shape = None if bias is None else tuple(bias.shape)
        _save(ctx, probs, factor, key_lengths)
        return dropped

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_upper_triang_masked_softmax_cuda as kernels

        probs, factor, key_lengths = _saved(ctx)
        prob, seed, window, zero_block = ctx.conf
        grad = kernels.backward_dropout(output_grads, probs, factor[0], prob, seed, window, zero_block, key_lengths)
        grad_bias = None
        if ctx.bias_shape is not None and ctx.needs_input_grad[7]:
            full = grad
            if zero_block:
                sq = ctx.bias_shape[-2]
                full = torch.where(_written_blocks(sq, zero_block, window, grad.device), grad, torch.zeros_like(grad))
            grad_bias = _batch_sum(full, ctx.bias_shape)
        return grad, None, None, None, None, None, None, grad_bias, None, None


class ScaledMaskedSoftmax(torch.autograd.Function):
    """``softmax(where(mask, -10000, scale * x))`` over the last dimension of
    ``[b, np, sq, sk]`` scores with a ``[1 or b, 1, sq, sk]`` mask.

    ``alibi_slopes``, ``bias`` and ``key_lengths`` are optional extras (see
    ``scaled_masked_softmax_cuda.forward``); the reference signature is ``apply(inputs, mask, scale)``."""

    @staticmethod
    def forward(ctx, inputs, mask, scale, alibi_slopes=None, bias=None, key_lengths=None, narrow_scale=False):
        import scaled_masked_softmax_cuda as kernels

        factor = _scale_tensor(scale)
        out = kernels.forward(inputs, mask, factor[0], alibi_slopes, bias, key_lengths, narrow_scale=narrow_scale)
        ctx.bias_shape = None if bias is None else tuple(bias.shape)
        ctx.save_for_backward(out, factor)
        return out

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_masked_softmax_cuda as kernels

        out, factor = ctx.saved_tensors
        grad = kernels.backward(output_grads, out, factor[0])
        grad_bias = None
        if ctx.bias_shape is not None and ctx.needs_input_grad[4]:
            grad_bias = _batch_sum(grad, ctx.bias_shape)
        return grad, None, None, None, grad_bias, None, None


class ScaledMaskedSoftmaxDropout(torch.autograd.Function):
    """``dropout(softmax(where(mask, -10000, scale * x)))`` in one kernel forward and one backward.
    No counterpart in the reference, which runs ``torch.nn.Dropout`` on the probabilities."""

    @staticmethod
    def forward(ctx, inputs, mask, scale, prob, seed, alibi_slopes=None, bias=None, key_lengths=None,
                narrow_scale=False):
        import scaled_masked_softmax_cuda as kernels

        factor = _scale_tensor(scale)
        dropped, probs = kernels.forward_dropout(inputs, mask, factor[0], prob, seed, alibi_slopes, bias, key_lengths,
                                                 narrow_scale=narrow_scale)
        ctx.conf = (float(prob), int(seed))
        ctx.bias_shape = None if bias is None else tuple(bias.shape)
        ctx.save_for_backward(probs, factor)
        return dropped

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_masked_softmax_cuda as kernels

        probs, factor = ctx.saved_tensors
        prob, seed = ctx.conf
        grad = kernels.backward_dropout(output_grads, probs, factor[0], prob, seed)
        grad_bias = None
        if ctx.bias_shape is not None and ctx.needs_input_grad[6]:
            grad_bias = _batch_sum(grad, ctx.bias_shape)
        return grad, None, None, None, None, None, grad_bias, None, None


class FusedScaleMaskSoftmax(nn.Module):
    """Scaling, masking and softmax of attention scores ``[b, np, sq, sk]``.

    Arguments:
        input_in_fp16: the scores are fp16.
        input_in_bf16: the scores are bf16.
        fusion_type: a ``SoftmaxFusionTypes`` member; ``none`` always takes the
            torch branch.
        mask_func: ``mask_func(scores, mask)``, used by the torch branch.
        softmax_in_fp32: run the torch branch in fp32.
        scale: factor applied to the scores before the softmax, or None.
        sliding_window_width: (extension) with ``upper_triang`` fusion, row q
            attends to keys q-width..q only, applied inside the kernel. The mask
            given to ``forward`` must then be the sliding-window mask, which is
            what the torch branch uses.
        alibi_slopes: (extension) fp32 tensor ``[np]``; the AliBi bias is added
            inside the causal kernel, and by the other branches with the same
            roundings, so the caller must not add it.
        attention_dropout: (extension) dropout probability applied to the
            probabilities in training mode; fused with the softmax on both
            kernel branches, whatever else (bias, AliBi, key lengths) is in play.
            The caller must not apply its own dropout.
        narrow_forward_scale: (extension, default False) on the fused branches round ``scale`` to
            the scores' dtype before the forward kernel uses it, which is what the reference's CUDA
            forward dispatchers do (``const input_t scale``, scaled_upper_triang_masked_softmax.h:368,
            scaled_masked_softmax.h:358). True: results follow the reference's fused kernels.
            False: the fp32 value is used, results follow the reference's torch branch
            (``forward_torch_softmax``). The backward uses the fp32 value either way, as the
            reference's does. Only factors that are not representable in the scores' dtype differ:
            1/sqrt(128) becomes 0.08837890625 (1.07e-4 smaller), 1/sqrt(64) is exact.
    """

    def __init__(self, input_in_fp16, input_in_bf16, fusion_type, mask_func, softmax_in_fp32, scale,
                 sliding_window_width=None, alibi_slopes=None, attention_dropout=0.0, narrow_forward_scale=False):
        super().__init__()
        assert isinstance(fusion_type, SoftmaxFusionTypes), f"Invalid fusion type {fusion_type}"
        assert scale is None or softmax_in_fp32, "softmax should be in fp32 when scaled"

        self.fusion = fusion_type is not SoftmaxFusionTypes.none
        if self.fusion:
            load_fused_kernels()  # leaves the process if the kernels are not installed
        self.upper_triang_mask_fusion = fusion_type is SoftmaxFusionTypes.upper_triang
        self.general_mask_fusion = fusion_type is SoftmaxFusionTypes.general

        self.input_in_fp16 = input_in_fp16
        self.input_in_bf16 = input_in_bf16
        self.input_in_float16 = bool(input_in_fp16 or input_in_bf16)
        self.softmax_in_fp32 = softmax_in_fp32
        self.mask_func = mask_func
        self.scale = scale

        assert 0.0 <= attention_dropout < 1.0, "attention_dropout must be in [0, 1)"
        self.attention_dropout = float(attention_dropout)
        self.narrow_forward_scale = bool(narrow_forward_scale)
        self.sliding_window_width = sliding_window_width
        if alibi_slopes is None:
            self.alibi_slopes = None
        else:
            self.register_buffer("alibi_slopes", alibi_slopes.detach().float().clone(), persistent=False)

    # ------------------------------------------------------------------ dispatch
    def forward(self, input, mask, bias=None, key_lengths=None):
        return self._dispatch(input, mask, bias, key_lengths, 0)

    def _forward_block_limited(self, input, mask, bias, key_lengths, zero_block):
        """For a caller that reads the probabilities (and their gradient) only in square blocks of ``zero_block``
        rows and columns and skips the blocks without a visible (query, key) pair: the causal kernel then leaves
        those blocks of its results UNWRITTEN (see ``scaled_upper_triang_masked_softmax_cuda.forward``); the other
        branches ignore the hint. Not part of the module's public surface: a dense consumer of the result would
        read uninitialised memory."""
        return self._dispatch(input, mask, bias, key_lengths, zero_block)

    def _dispatch(self, input, mask, bias, key_lengths, zero_block):
        assert input.dim() == 4  # [b, np, sq, sk]
        dropout = self.attention_dropout if self.training else 0.0
        if self.upper_triang_mask_fusion and input.size(2) != input.size(3):
            # the last rows of a longer causal matrix (new positions after cached keys): the triangle the causal
            # kernel implies does not apply, the caller's mask does. The reference asserts sq == sk here
            # (fused_softmax.py:173) when its gate lets such a shape through.
            if self._rectangular_kernel_available(mask, *input.size()):
                return self._forward_general(input, mask, bias, key_lengths, dropout)
        elif self.is_kernel_available(mask, *input.size()):
            return self.forward_fused_softmax(input, mask, bias, key_lengths, zero_block, dropout)
        probs = self.forward_torch_softmax(input, mask, bias, key_lengths)
        if dropout > 0.0:
            probs = torch.nn.functional.dropout(probs, p=dropout, training=True)
        return probs

    def _rectangular_kernel_available(self, mask, b, np, sq, sk):
        return (self.input_in_float16 and mask is not None and sk > 16 and sq % 4 == 0 and (b * np) % 4 == 0
                and sq % self.get_batch_per_block(sq, sk, b, np) == 0 and self.alibi_slopes is None)

    def is_kernel_available(self, mask, b, np, sq, sk):
        """The reference's conditions (fused_softmax.py:148-168) without ``sk <= 2048``."""
        if not self.fusion or not self.input_in_float16 or mask is None:
            return False
        attn_batches = b * np
        if sk <= 16 or sq % 4 or attn_batches % 4:
            return False
        rows_per_block = self.get_batch_per_block(sq, sk, b, np)
        divided = attn_batches if self.upper_triang_mask_fusion else sq
        return divided % rows_per_block == 0

    @staticmethod
    def get_batch_per_block(sq, sk, b, np):
        import scaled_masked_softmax_cuda

        return scaled_masked_softmax_cuda.get_batch_per_block(sq, sk, b, np)

    # ------------------------------------------------------------------ branches
    @staticmethod
    def _mask_with_padding(mask, key_lengths, b, sk):
        """The mask with the padding keys ``k >= key_lengths[b]`` added: ``[b, 1, sq, sk]``."""
        if key_lengths is None:
            return mask
        assert key_lengths.shape == (b,), "key_lengths must be [b]"
        keys = torch.arange(sk, device=mask.device)
        padding = keys.view(1, 1, 1, sk) >= key_lengths.to(mask.device).view(b, 1, 1, 1)
        return (mask.bool() | padding).contiguous()

    @staticmethod
    def _dropout_seed(device):
        # from the device's CUDA generator, read on the host: follows torch.manual_seed, no synchronisation
        return dropout_rng.next_seed(device)

    def _slopes_on(self, device):
        slopes = self.alibi_slopes
        if slopes is not None and slopes.device != device:
            slopes = slopes.to(device)
        return slopes

    def _forward_general(self, input, mask, bias, key_lengths, dropout):
        """The padding-mask kernel; bias, AliBi, key lengths and dropout all happen inside it."""
        b, np, sq, sk = input.size()
        factor = 1.0 if self.scale is None else self.scale
        if bias is not None:
            assert bias.shape[-3:] == (np, sq, sk) and bias.numel() == np * sq * sk, "bias must be [1, np, sq, sk]"
        if key_lengths is not None:
            assert key_lengths.shape == (b,), "key_lengths must be [b]"
        slopes = self._slopes_on(input.device)
        if dropout > 0.0:
            return ScaledMaskedSoftmaxDropout.apply(input, mask, factor, dropout, self._dropout_seed(input.device), slopes, bias,
                                                    key_lengths, self.narrow_forward_scale)
        return ScaledMaskedSoftmax.apply(input, mask, factor, slopes, bias, key_lengths, self.narrow_forward_scale)

    def forward_fused_softmax(self, input, mask, bias=None, key_lengths=None, zero_block=0, dropout=0.0):
        b, np, sq, sk = input.size()
        factor = 1.0 if self.scale is None else self.scale
        if not self.upper_triang_mask_fusion:
            return self._forward_general(input, mask, bias, key_lengths, dropout)

        assert sq == sk, "causal mask is only for self attention"
        slopes = self._slopes_on(input.device)
        # the kernel takes [attn_batches, sq, sk]; the causal mask is implied by the indices
        flat = input.view(b * np, sq, sk)
        if bias is not None:
            assert bias.shape[-3:] == (np, sq, sk) and bias.numel() == np * sq * sk, "bias must be [1, np, sq, sk]"
        if key_lengths is not None:
            assert key_lengths.shape == (b,), "key_lengths must be [b]"
        if dropout > 0.0:
            probs = ScaledUpperTriangMaskedSoftmaxDropout.apply(flat, factor, dropout, self._dropout_seed(input.device),
                                                                self.sliding_window_width, zero_block, slopes, bias,
                                                                key_lengths, self.narrow_forward_scale)
        else:
            probs = ScaledUpperTriangMaskedSoftmax.apply(flat, factor, self.sliding_window_width, slopes, bias,
                                                         key_lengths, zero_block, self.narrow_forward_scale)
        return probs.view(b, np, sq, sk)

    def forward_torch_softmax(self, input, mask, bias=None, key_lengths=None):
        if key_lengths is not None and mask is not None:
            mask = self._mask_with_padding(mask, key_lengths, input.size(0), input.size(3))
        if bias is not None:
            input = input + bias
        if self.alibi_slopes is not None:
            input = self._add_alibi(input)
        widen = self.input_in_float16 and self.softmax_in_fp32
        work = input.float() if widen else input
        if self.scale is not None:
            work = work * self.scale
        if mask is not None:
            work = self.mask_func(work, mask)
        probs = torch.nn.Softmax(dim=-1)(work)
        if widen:
            probs = probs.half() if self.input_in_fp16 else probs.bfloat16()
        return probs

    def _add_alibi(self, scores):
        """``scores + alibi_matrix`` in the scores' dtype for sq == sk, with the arithmetic of
        ``AliBi.forward`` (megatron/model/positional_embeddings.py:219-257)."""
        s = scores.shape[-1]
        assert scores.shape[-2] == s, "in-module AliBi needs sq == sk"
        pos = torch.arange(s, device=scores.device)
        distance = -torch.tril(pos.view(s, 1) - pos.view(1, s)).to(scores.dtype)
        slopes = self.alibi_slopes.to(scores.device).to(scores.dtype)
        return scores + distance * slopes.view(-1, 1, 1)
