"""The one function of the reference's ``megatron/model/utils.py`` that belongs to the fused softmax path:
the choice of the fusion type from the two configuration flags (:356-362), which the attention layer
hands to ``FusedScaleMaskSoftmax`` (megatron/model/transformer.py:449-455)."""
from .fused_softmax import SoftmaxFusionTypes

__all__ = ["get_fusion_type"]


def get_fusion_type(neox_args):
    """``upper_triang`` when ``scaled_upper_triang_masked_softmax_fusion`` is set (it wins over the other flag),
    ``general`` when only ``scaled_masked_softmax_fusion`` is, ``none`` otherwise."""
    if neox_args.scaled_upper_triang_masked_softmax_fusion:
        return SoftmaxFusionTypes.upper_triang
    if neox_args.scaled_masked_softmax_fusion:
        return SoftmaxFusionTypes.general
    return SoftmaxFusionTypes.none
