"""One transformer layer on one GPU, assembled from the kernels of libneox_hotpath.so.

The data flow of GPT-NeoX's ``ParallelTransformerLayer`` (megatron/model/transformer.py:962-1321)
with ``ParallelSelfAttention`` (:326-959) and ``ParallelMLP`` (:93-196) inside, without the
model-parallel layers: every linear layer is a plain ``torch.nn.functional.linear`` (library
GEMM) that hands its bias on instead of adding it (``skip_bias_add``), and everything between
the GEMMs is one of the fused kernels:

    norm                      nhp_layernorm / nhp_rmsnorm (the two norms of the parallel-residual layout: nhp_layernorm_pair)
    qkv projection            GEMM (bias added by the GEMM, as ColumnParallelLinear does for qkv)
    rotary on q and k         nhp_rope_cached_qk on the two views of the projection output; its backward writes
                              into the gradient of the projection output (no concatenation)
    scores / probs / context  CoreAttention: GEMM, fused softmax (+ dropout), GEMM
    output projection         GEMM, bias handed on
    bias + dropout + residual nhp_bias_add_residual / nhp_bias_dropout_add
    MLP                       GEMM, bias+GeLU or gated activation kernel, GEMM, bias handed on

Both residual layouts of the reference are provided: the sequential one
(``x = x + attn(ln1(x)); x = x + mlp(ln2(x))``, :1254-1318) and the parallel one of the
GPT-J / Pythia configurations (``x = x + attn(ln1(x)) + mlp(ln2(x))``, :1195-1250).
With ``use_cache`` a layer keeps the keys and values of the positions seen so far (``layer_past``) and the
next call continues after them (inference, :916-935). Left out: tensor / sequence / pipeline parallelism,
mixture of experts, flash and sparse attention, Transformer Engine layers.
"""
import torch
import torch.nn.functional as F

from .activations import Gated_Activation, get_activation
from .attention_core import (CoreAttention, apply_rotary_to_query_key, get_fusion_type, split_gqa_and_rotate,
                             split_qkv_and_rotate)
from .fused_bias_dropout import (bias_add_residual_pair, bias_dropout_add_fused_inference, bias_dropout_add_fused_train,
                                 get_bias_dropout_add)
from .norms import get_norm, layer_norm_pair
from .positional_embeddings import AliBi, RotaryEmbedding


class Linear(torch.nn.Module):
    """``y = x W^T (+ b)``; with ``skip_bias_add`` the bias is returned beside the product instead of being
    added (what the reference's Column/RowParallelLinear do, megatron/mpu/layers.py), so that the next fused
    kernel can add it."""

    def __init__(self, input_size, output_size, bias=True, skip_bias_add=False, std=0.02):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.empty(output_size, input_size))
        torch.nn.init.normal_(self.weight, mean=0.0, std=std)
        self.bias = torch.nn.Parameter(torch.zeros(output_size)) if bias else None
        self.skip_bias_add = skip_bias_add

    def forward(self, x):
        if self.skip_bias_add:
            return F.linear(x, self.weight), self.bias
        return F.linear(x, self.weight, self.bias), None


class MLP(torch.nn.Module):
    """``ParallelMLP`` (megatron/model/transformer.py:93-196): h -> ffn -> activation -> h, the second bias handed on."""

    def __init__(self, neox_args, multiple_of=256):
        super().__init__()
        self.activation_func, self.is_gated = get_activation(neox_args)
        self.activation_type = neox_args.activation
        self.bias_gelu_fusion = getattr(neox_args, "bias_gelu_fusion", False)
        hidden = neox_args.hidden_size
        if getattr(neox_args, "intermediate_size", None):
            ffn_dim = neox_args.intermediate_size
        elif getattr(neox_args, "expansion_factor", None):
            ffn_dim = int(neox_args.expansion_factor * hidden)
        else:
            ffn_dim = 4 * hidden
        ffn_dim_in = ffn_dim
        if self.is_gated:
            self.activation_func = Gated_Activation(self.activation_func)
            ffn_dim = int(ffn_dim * 2 / 3)   # a gated MLP of equal parameter count
            ffn_dim_in = ffn_dim // 2
        ffn_dim = int((2 * multiple_of) * ((ffn_dim + 2 * multiple_of - 1) // (2 * multiple_of)))
        ffn_dim_in = int(multiple_of * ((ffn_dim_in + multiple_of - 1) // multiple_of))
        use_bias = getattr(neox_args, "use_bias_in_mlp", True)
        self.linear1 = Linear(hidden, ffn_dim, bias=use_bias, skip_bias_add=True)
        self.linear2 = Linear(ffn_dim_in, hidden, bias=use_bias, skip_bias_add=True)

    def forward(self, hidden_states):
        intermediate, bias = self.linear1(hidden_states)
        if self.is_gated or (self.activation_type == "gelu" and self.bias_gelu_fusion):
            if bias is None and not self.is_gated:
                bias = torch.zeros(intermediate.size(-1), dtype=intermediate.dtype, device=intermediate.device)
            intermediate = self.activation_func(intermediate, bias)
        else:
            intermediate = self.activation_func(intermediate if bias is None else intermediate + bias)
        return self.linear2(intermediate)


class SelfAttention(torch.nn.Module):
    """``ParallelSelfAttention`` (megatron/model/transformer.py:326-959) with the unfused ("global") attention:
    fused qkv projection, views split along the last dimension, rotary, CoreAttention, output projection.
    With ``num_kv_heads`` below ``num_attention_heads`` (grouped-query attention, ``gqa_project``, :768-839)
    the projection is ``[q heads | k heads | v heads]`` and the k/v heads are shared by groups of query heads
    without being repeated."""

    def __init__(self, neox_args, attention_mask_func, layer_number, rpe=None, rotary=False, use_cache=False):
        super().__init__()
        self.fp16 = neox_args.precision == "fp16"
        self.bf16 = neox_args.precision == "bfloat16"
        self.num_heads = neox_args.num_attention_heads
        self.head_dim = neox_args.hidden_size // self.num_heads
        self.pos_emb = neox_args.pos_emb
        use_bias = getattr(neox_args, "use_bias_in_attn_linear", True)
        self.num_kv_heads = getattr(neox_args, "num_kv_heads", None) or self.num_heads
        assert self.num_heads % self.num_kv_heads == 0, "num_kv_heads must divide num_attention_heads"
        self.gqa = self.num_kv_heads != self.num_heads
        self.query_key_value = Linear(neox_args.hidden_size, (self.num_heads + 2 * self.num_kv_heads) * self.head_dim,
                                      bias=use_bias)
        slopes = AliBi(self.num_heads, 1, 0).slopes if self.pos_emb == "alibi" else None
        self.rotary_ndims = None
        self.rotary_emb = None
        if rotary:
            pct = getattr(neox_args, "rotary_pct", 1.0)
            if pct != 1:
                self.rotary_ndims = int(self.head_dim * pct)
            dtype = torch.float16 if self.fp16 else torch.bfloat16 if self.bf16 else torch.float32
            self.rotary_emb = RotaryEmbedding(self.rotary_ndims or self.head_dim, base=getattr(neox_args, "rotary_emb_base", 10000),
                                              max_seq_len=neox_args.seq_length, precision=dtype)
        self.rope_fusion = getattr(neox_args, "rope_fusion", True)
        self.core = CoreAttention(
            self.head_dim, layer_number, self.fp16, self.bf16, get_fusion_type(neox_args), attention_mask_func,
            attention_softmax_in_fp32=getattr(neox_args, "attention_softmax_in_fp32", False),
            apply_query_key_layer_scaling=getattr(neox_args, "apply_query_key_layer_scaling", False),
            use_mup=getattr(neox_args, "use_mup", False), attention_dropout=getattr(neox_args, "attention_dropout", 0.0),
            sliding_window_width=getattr(neox_args, "sliding_window_width", None), alibi_slopes=slopes, rpe=rpe,
            use_cache=use_cache)
        self.use_cache = use_cache
        self.dense = Linear(neox_args.hidden_size, neox_args.hidden_size, bias=use_bias, skip_bias_add=True)

    def forward(self, hidden_states, attention_mask, layer_past=None):
        """Returns ``(output, bias)``; with ``use_cache`` the first item is ``[output, present]``, ``present`` the
        stacked keys and values of all positions so far (megatron/model/transformer.py:916-958). ``layer_past``:
        the ``present`` of the previous call; the rotary embedding then starts at the position after it and
        ``attention_mask`` must hold the rows of the new positions over all keys."""
        sq, b = hidden_states.size(0), hidden_states.size(1)
        mixed, _ = self.query_key_value(hidden_states)
        if self.gqa:
            query, key, value = self._gqa_project(mixed, layer_past)
        else:
            # [sq, b, np * 3 * hn] -> [sq, b, np, 3 * hn] -> three views [sq, b, np, hn]
            mixed = mixed.view(sq, b, self.num_heads, 3 * self.head_dim)
            if self.rotary_emb is not None and self.rope_fusion:
                query, key, value = split_qkv_and_rotate(mixed, self.rotary_emb, layer_past=layer_past)
            else:
                query, key, value = torch.split(mixed, self.head_dim, dim=-1)
                if self.rotary_emb is not None:
                    query, key = apply_rotary_to_query_key(query, key, self.rotary_emb, rotary_ndims=self.rotary_ndims,
                                                           rope_fusion=False, bf16=self.bf16, layer_past=layer_past)
        if layer_past is not None and layer_past.numel() > 0:
            past_key, past_value = layer_past
            key = torch.cat((past_key.type_as(key), key), dim=0)
            value = torch.cat((past_value.type_as(value), value), dim=0)
        present = torch.stack((key, value)) if self.use_cache else None
        # [sq, b, np * hn], written in that layout by the context GEMM
        context = self.core(query, key, value, attention_mask, merged_heads=True)
        output, bias = self.dense(context)
        return ([output, present] if self.use_cache else output), bias

    def _gqa_project(self, mixed, layer_past=None):
        """``[sq, b, (np + 2 * nkv) * hn]`` -> q ``[sq, b, np, hn]``, k and v ``[sq, b, nkv, hn]``, q and k rotated."""
        sq, b = mixed.shape[:2]
        np_, nkv, hn = self.num_heads, self.num_kv_heads, self.head_dim
        if self.rotary_emb is not None and self.rope_fusion:
            return split_gqa_and_rotate(mixed, self.rotary_emb, np_, nkv, layer_past=layer_past)
        query, key, value = torch.split(mixed, (np_ * hn, nkv * hn, nkv * hn), dim=-1)
        query, key, value = query.view(sq, b, np_, hn), key.view(sq, b, nkv, hn), value.view(sq, b, nkv, hn)
        if self.rotary_emb is not None:
            query, key = apply_rotary_to_query_key(query, key, self.rotary_emb, rotary_ndims=self.rotary_ndims,
                                                   rope_fusion=False, bf16=self.bf16, layer_past=layer_past)
        return query, key, value


class TransformerLayer(torch.nn.Module):
    """``ParallelTransformerLayer.forward`` (megatron/model/transformer.py:1179-1321) on one GPU.
    Input and output ``[s, b, h]``."""

    def __init__(self, neox_args, attention_mask_func, layer_number, rpe=None, rotary=False, use_cache=False):
        super().__init__()
        norm, eps = get_norm(neox_args)
        self.input_layernorm = norm(neox_args.hidden_size, eps=eps)
        self.post_attention_layernorm = norm(neox_args.hidden_size, eps=eps)
        self.hidden_dropout = getattr(neox_args, "hidden_dropout", 0.0)
        self.bias_dropout_fusion = getattr(neox_args, "bias_dropout_fusion", True)
        self.gpt_j_residual = getattr(neox_args, "gpt_j_residual", False)
        self.gpt_j_tied = getattr(neox_args, "gpt_j_tied", False)
        self.use_cache = use_cache
        self.layer_past = None   # with use_cache: keys and values after the last call (transformer.py:1166, 1219-1225)
        self.attention = SelfAttention(neox_args, attention_mask_func, layer_number, rpe=rpe, rotary=rotary,
                                       use_cache=use_cache)
        self.mlp = MLP(neox_args)

    def _get_bias_dropout(self):
        if self.bias_dropout_fusion:
            return bias_dropout_add_fused_train if self.training else bias_dropout_add_fused_inference
        return get_bias_dropout_add(self.training)

    def _attend(self, x, attention_mask, layer_past):
        output, bias = self.attention(x, attention_mask, layer_past=layer_past)
        if self.use_cache:
            output, self.layer_past = output
        return output, bias

    def forward(self, x, attention_mask, layer_past=None):
        layer_past = layer_past if layer_past is not None else self.layer_past
        bias_dropout_fn = self._get_bias_dropout()
        residual = x
        if self.gpt_j_residual:
            # x = x + attn(ln1(x)) + mlp(ln2(x))
            if self.gpt_j_tied:
                x1 = x2 = self.input_layernorm(x)
            else:
                x1, x2 = layer_norm_pair(x, self.input_layernorm, self.post_attention_layernorm)
            attention_output, attention_bias = self._attend(x1, attention_mask, layer_past)
            if self.bias_dropout_fusion and (self.hidden_dropout == 0.0 or not self.training):
                # no dropout: attention branch + MLP branch + residual in one pass
                mlp_output, mlp_bias = self.mlp(x2)
                return bias_add_residual_pair(attention_output, attention_bias, mlp_output, mlp_bias, residual)
            if attention_bias is not None:
                attention_output = bias_dropout_fn(attention_output, bias=attention_bias, residual=None,
                                                   prob=self.hidden_dropout)
            mlp_output, mlp_bias = self.mlp(x2)
            output = bias_dropout_fn(mlp_output, bias=mlp_bias, residual=attention_output, prob=self.hidden_dropout)
            return bias_dropout_add_fused_inference(output, None, residual, 0.0)  # residual + output
        # x = x + attn(ln1(x)); x = x + mlp(ln2(x))
        attention_output, attention_bias = self._attend(self.input_layernorm(x), attention_mask, layer_past)
        attention_output = bias_dropout_fn(attention_output, bias=attention_bias, residual=residual,
                                           prob=self.hidden_dropout)
        mlp_output, mlp_bias = self.mlp(self.post_attention_layernorm(attention_output))
        return bias_dropout_fn(mlp_output, bias=mlp_bias, residual=attention_output, prob=self.hidden_dropout)
