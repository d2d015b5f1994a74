"""Hot-path subset of ``megatron.model``. Exported here: the fused scale-mask-softmax, the fused rotary
embedding and the rotary cache. Submodules, imported by name as in the reference: ``activations`` (bias+GeLU,
gated activations), ``fused_bias_dropout``, ``norms`` and ``fused_layer_norm`` (the neighbouring
bandwidth-bound kernels of the layer), ``utils`` (``get_fusion_type``), ``dropout_rng``, and the single-GPU
callers ``attention_core``, ``transformer_layer`` and ``gmlp`` that put the kernels to use. No model zoo, no
parallel layers."""
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
