"""Scale + mask + softmax for attention scores, with the same public surface as
GPT-NeoX's ``megatron/model/fused_softmax.py``:

  ScaledUpperTriangMaskedSoftmax (:24-53), ScaledMaskedSoftmax (:56-83),
  SoftmaxFusionTypes (:86-89), FusedScaleMaskSoftmax (:92-205).

The fused paths call the gfx950 kernels through the extension-module names the
reference uses. Differences from the reference, all widening:
  * the fused path takes key lengths above 2048 (the kernels keep rows of up
    to 65536 keys in registers, longer ones stream);
  * ``scale`` reaches the forward kernel as an fp32 value; the reference's CUDA
    dispatcher first narrows it to the input dtype.
"""
import enum

import torch
import torch.nn as nn

from ..fused_kernels import load_fused_kernels


class ScaledUpperTriangMaskedSoftmax(torch.autograd.Function):
    """softmax(scale * x) under a causal (upper-triangular) mask on a
    [attn_batches, sq, sk] tensor, fused into one kernel each way."""

    @staticmethod
    def forward(ctx, inputs, scale):
        import scaled_upper_triang_masked_softmax_cuda as ext

        scale_t = torch.tensor([scale])
        probs = ext.forward(inputs, scale_t[0])
        ctx.save_for_backward(probs, scale_t)
        return probs

    @staticmethod
    def backward(ctx, output_grads):
        import scaled_upper_triang_masked_softmax_cuda as ext

        probs, scale_t = ctx.saved_tensors
        return ext.backward(output_grads, probs, scale_t[0]), None


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
    """

    def __init__(self, input_in_fp16, input_in_bf16, fusion_type, mask_func, softmax_in_fp32, scale):
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
            probs = ScaledUpperTriangMaskedSoftmax.apply(input.view(-1, sq, sk), scale)
            return probs.view(b, np, sq, sk)
        return ScaledMaskedSoftmax.apply(input, mask, scale)

    def forward_torch_softmax(self, input, mask):
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
