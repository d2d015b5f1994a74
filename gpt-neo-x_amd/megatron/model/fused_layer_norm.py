"""The fused LayerNorm / RMSNorm classes of GPT-NeoX on MI355X.

Surface of ``megatron/model/fused_layer_norm.py``: ``MixedFusedLayerNorm`` (:34-153) and
``MixedFusedRMSNorm`` (:156-262), which the reference backs with apex's
``fused_layer_norm_cuda``. Here both run on the hand-written gfx950 kernels of
libneox_hotpath.so (the same ones as ``norms.LayerNorm`` / ``norms.RMSNorm``); there is
no separate "persistent" kernel, so ``no_persist_layer_norm`` and the ``mem_efficient_*``
switches are accepted and stored but select nothing. Parameter names (``weight`` / ``bias``,
``scale``), their ``sequence_parallel`` attribute and the ``*_1p`` convention (the stored
parameter is the weight minus one) are the reference's.
"""
import numbers

import torch

from .norms import _LayerNormFunction, _RMSNormFunction


def _shape_of(normalized_shape):
    if isinstance(normalized_shape, numbers.Integral):
        normalized_shape = (int(normalized_shape),)
    shape = torch.Size(normalized_shape)
    if len(shape) != 1:
        raise NotImplementedError("only normalisation over the last dimension is provided")
    return shape


class MixedFusedLayerNorm(torch.nn.Module):
    def __init__(self, normalized_shape, eps=1e-5, no_persist_layer_norm=True, sequence_parallel=False,
                 apply_layernorm_1p=False, mem_efficient_ln=True):
        super().__init__()
        self.apply_layernorm_1p = apply_layernorm_1p
        self.mem_efficient_ln = mem_efficient_ln
        self.normalized_shape = _shape_of(normalized_shape)
        self.eps = eps
        self.weight = torch.nn.Parameter(torch.empty(*self.normalized_shape))
        self.bias = torch.nn.Parameter(torch.empty(*self.normalized_shape))
        self.reset_parameters()
        self.no_persist_layer_norm = no_persist_layer_norm
        self.sequence_parallel = sequence_parallel
        setattr(self.weight, "sequence_parallel", self.sequence_parallel)
        setattr(self.bias, "sequence_parallel", self.sequence_parallel)

    def reset_parameters(self):
        if self.apply_layernorm_1p:
            torch.nn.init.zeros_(self.weight)
        else:
            torch.nn.init.ones_(self.weight)
        torch.nn.init.zeros_(self.bias)

    def forward(self, input):
        if input.size(-1) != self.normalized_shape[0]:
            raise RuntimeError(f"MixedFusedLayerNorm: expected last dimension {self.normalized_shape[0]}, "
                               f"got {input.size(-1)}")
        weight = self.weight + 1 if self.apply_layernorm_1p else self.weight
        return _LayerNormFunction.apply(input, weight, self.bias, self.eps)


class MixedFusedRMSNorm(torch.nn.Module):
    """``scale * x * rsqrt(mean(x^2) + eps)``."""

    def __init__(self, normalized_shape, eps=1e-5, no_persist_layer_norm=True, sequence_parallel=False,
                 apply_rmsnorm_1p=False, mem_efficient_rms=True):
        super().__init__()
        self.apply_rmsnorm_1p = apply_rmsnorm_1p
        self.mem_efficient_rms = mem_efficient_rms
        self.normalized_shape = _shape_of(normalized_shape)
        self.eps = eps
        self.scale = torch.nn.Parameter(torch.empty(*self.normalized_shape))
        self.reset_parameters()
        self.no_persist_layer_norm = no_persist_layer_norm
        self.sequence_parallel = sequence_parallel
        setattr(self.scale, "sequence_parallel", self.sequence_parallel)

    def reset_parameters(self):
        if self.apply_rmsnorm_1p:
            torch.nn.init.zeros_(self.scale)
        else:
            torch.nn.init.ones_(self.scale)

    def forward(self, input):
        if input.size(-1) != self.normalized_shape[0]:
            raise RuntimeError(f"MixedFusedRMSNorm: expected last dimension {self.normalized_shape[0]}, "
                               f"got {input.size(-1)}")
        weight = self.scale + 1 if self.apply_rmsnorm_1p else self.scale
        return _RMSNormFunction.apply(input, weight, None, self.eps, 0, None)
