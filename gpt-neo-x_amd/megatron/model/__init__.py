"""Hot-path subset of ``megatron.model``: fused scale-mask-softmax, fused rotary
embedding and the rotary cache. Nothing else of the model zoo lives here."""
from .fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes
from .fused_rope import (
    fused_apply_rotary_pos_emb,
    fused_apply_rotary_pos_emb_cached,
    fused_apply_rotary_pos_emb_qk_cached,
)
from .positional_embeddings import (
    AliBi,
    RotaryEmbedding,
    apply_rotary_pos_emb,
    apply_rotary_pos_emb_torch,
    rotate_half,
)
