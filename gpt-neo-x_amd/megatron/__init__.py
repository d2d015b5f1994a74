"""Drop-in subset of the GPT-NeoX ``megatron`` package: the fused softmax / rotary hot path
(``megatron.fused_kernels``, ``megatron.model.fused_softmax``, ``megatron.model.fused_rope``,
``megatron.model.positional_embeddings``) and its bandwidth-bound neighbours in the transformer layer
(``megatron.model.{activations,fused_bias_dropout,norms,fused_layer_norm}``), backed by hand-written
gfx950 kernels in ``libneox_hotpath.so``."""
