"""Drop-in subset of the GPT-NeoX ``megatron`` package: only the fused softmax /
rotary hot path (``megatron.fused_kernels``, ``megatron.model.fused_softmax``,
``megatron.model.fused_rope``, ``megatron.model.positional_embeddings``),
backed by hand-written gfx950 kernels in ``libneox_hotpath.so``."""
