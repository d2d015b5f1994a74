"""``get_fusion_type`` under the module path of the reference (megatron/model/utils.py:356-362)."""
from .attention_core import get_fusion_type

__all__ = ["get_fusion_type"]
