"""Scale + mask + softmax for attention scores, with the same public surface as
GPT-NeoX's ``megatron/model/fused_softmax.py``:

  ScaledUpperTriangMaskedSoftmax (:24-53), ScaledMaskedSoftmax (:56-83),
  SoftmaxFusionTypes (:86-89), FusedScaleMaskSoftmax (:92-205).

The fused paths call the gfx950 kernels through the extension-module names the
reference uses. Differences from the reference, all widening:
  * the fused path takes key lengths above 2048 (the kernels keep rows of up
    to 65536 keys in registers, longer ones stream);
  * ``scale`` reaches the forward kernel as an fp32 value; the reference's CUDA
    dispatcher first narrows it to the input dtype;
  * two optional constructor arguments of ``FusedScaleMaskSoftmax`` let the
    causal kernel do by index what its caller otherwise does with tensors:
    ``sliding_window_width`` (the reference's causal kernel ignores the mask
    contents and so drops a sliding window) and ``alibi_slopes`` (the AliBi
    bias is added inside the kernel instead of by a separate
    ``scores + alibi_matrix`` pass). Both default to off.
"""
import enum

import torch
import torch.nn as nn

from ..fused_kernels import load_fused_kernels


class ScaledUpperTriangMaskedSoftmax(torch.autograd.Function):
    """softmax(scale * x) under a causal (upper-triangular) mask on a
    [attn_batches, sq, sk] tensor, fused into one kernel each way."""

    @staticmethod
    def forward(ctx, inputs, scale, window=None, alibi_slopes=None):
        import scaled_upper_triang_masked_softmax_cuda as ext

        scale_t = torch.tensor([scale])
        probs = ext.forward(inputs, scale_t[0], window, alibi_slopes)
        ctx.save_for_backward(probs, scale_t)
        ctx.window = window
        return probs

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_upper_triang_masked_softmax_cuda as ext

        probs, scale_t = ctx.saved_tensors
        return ext.backward(output_grads, probs, scale_t[0], ctx.window), None, None, None


class ScaledMaskedSoftmax(torch.autograd.Function):
    """softmax(where(mask, -10000, scale * x)) on a [b, np, sq, sk] tensor,
    fused into one kernel each way."""

    @staticmethod
    def forward(ctx, inputs, mask, scale):
        import scaled_masked_softmax_cuda as ext

        scale_t = torch.tensor([scale])
        probs = ext.forward(inputs, mask, scale_t[0])
        ctx.save_for_backward(probs, scale_t)
        return probs

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_masked_softmax_cuda as ext

        probs, scale_t = ctx.saved_tensors
        return ext.backward(output_grads, probs, scale_t[0]), None, None


class SoftmaxFusionTypes(enum.Enum):
    upper_triang = 1  # causal mask
    general = 2  # general mask
    none = 3  # no fusion


class FusedScaleMaskSoftmax(nn.Module):
    """Scaling, masking and softmax of attention scores [b, np, sq, sk].

    Arguments:
        input_in_fp16: the scores are fp16.
        input_in_bf16: the scores are bf16.
        fusion_type: a SoftmaxFusionTypes member; ``none`` always takes the
            plain torch path.
        mask_func: ``mask_func(scores, mask)`` used by the torch path.
        softmax_in_fp32: compute the torch path in fp32.
        scale: factor applied to the scores before the softmax, or None.
        sliding_window_width: (extension) with upper_triang fusion, restrict row q
            to keys q-width..q inside the kernel. The mask handed to ``forward``
            must then be the sliding-window mask, which the torch path uses.
        alibi_slopes: (extension) fp32 tensor [np]; with upper_triang fusion the
            AliBi bias is added inside the kernel, and by the torch path with the
            same roundings, so the caller must not add it itself.
    """

    def __init__(self, input_in_fp16, input_in_bf16, fusion_type, mask_func, softmax_in_fp32, scale,
                 sliding_window_width=None, alibi_slopes=None):
        super().__init__()
        self.input_in_fp16 = input_in_fp16
        self.input_in_bf16 = input_in_bf16
        self.input_in_float16 = input_in_fp16 or input_in_bf16

        assert isinstance(fusion_type, SoftmaxFusionTypes), f"Invalid fusion type {fusion_type}"
        if fusion_type is not SoftmaxFusionTypes.none:
            load_fused_kernels()  # exits the process if the kernels are not installed

        self.upper_triang_mask_fusion = fusion_type is SoftmaxFusionTypes.upper_triang
        self.general_mask_fusion = fusion_type is SoftmaxFusionTypes.general
        self.fusion = fusion_type is not SoftmaxFusionTypes.none

        self.mask_func = mask_func
        self.softmax_in_fp32 = softmax_in_fp32
        self.scale = scale
        assert self.scale is None or softmax_in_fp32, "softmax should be in fp32 when scaled"

        self.sliding_window_width = sliding_window_width
        if alibi_slopes is not None:
            self.register_buffer("alibi_slopes", alibi_slopes.detach().float().clone(), persistent=False)
        else:
            self.alibi_slopes = None

    def forward(self, input, mask):
        assert input.dim() == 4  # [b, np, sq, sk]
        if self.is_kernel_available(mask, *input.size()):
            return self.forward_fused_softmax(input, mask)
        return self.forward_torch_softmax(input, mask)

    def is_kernel_available(self, mask, b, np, sq, sk):
        """The reference's gate (fused_softmax.py:148-168) without its
        ``sk <= 2048`` bound."""
        attn_batches = b * np
        if not (self.fusion and self.input_in_float16 and mask is not None):
            return False
        if not (sk > 16 and sq % 4 == 0 and attn_batches % 4 == 0):
            return False
        batch_per_block = self.get_batch_per_block(sq, sk, b, np)
        if self.upper_triang_mask_fusion:
            return attn_batches % batch_per_block == 0
        return sq % batch_per_block == 0

    def forward_fused_softmax(self, input, mask):
        b, np, sq, sk = input.size()
        scale = self.scale if self.scale is not None else 1.0
        if self.upper_triang_mask_fusion:
            assert sq == sk, "causal mask is only for self attention"
            # the causal kernel works on [attn_batches, sq, sk]; the mask is implied
            slopes = self.alibi_slopes
            if slopes is not None and slopes.device != input.device:
                slopes = slopes.to(input.device)
            probs = ScaledUpperTriangMaskedSoftmax.apply(
                input.view(-1, sq, sk), scale, self.sliding_window_width, slopes)
            return probs.view(b, np, sq, sk)
        if self.alibi_slopes is not None:
            input = self._add_alibi(input)
        return ScaledMaskedSoftmax.apply(input, mask, scale)

    def _add_alibi(self, scores):
        """scores + AliBi matrix in the scores' dtype, for sq == sk (the arithmetic of
        megatron/model/positional_embeddings.py:219-257)."""
        s = scores.shape[-1]
        assert scores.shape[-2] == s, "in-module AliBi needs sq == sk"
        i = torch.arange(s, device=scores.device)
        a = -torch.tril(i.view(s, 1) - i.view(1, s)).to(scores.dtype)
        slopes = self.alibi_slopes.to(scores.device).to(scores.dtype)
        return scores + a * slopes.view(-1, 1, 1)

    def forward_torch_softmax(self, input, mask):
        if self.alibi_slopes is not None:
            input = self._add_alibi(input)
        upcast = self.input_in_float16 and self.softmax_in_fp32
        if upcast:
            input = input.float()
        if self.scale is not None:
            input = input * self.scale
        masked = self.mask_func(input, mask) if mask is not None else input
        probs = torch.nn.Softmax(dim=-1)(masked)
        if upcast:
            probs = probs.half() if self.input_in_fp16 else probs.bfloat16()
        return probs

    @staticmethod
    def get_batch_per_block(sq, sk, b, np):
        import scaled_masked_softmax_cuda

        return scaled_masked_softmax_cuda.get_batch_per_block(sq, sk, b, np)
