"""gMLP / aMLP block on one GPU: the second caller of the fused softmax in GPT-NeoX.

``megatron/model/gmlp.py:28-141`` of the reference: a norm, an input projection to twice the
feed-forward width, the activation, the spatial gating unit (half of the features gate the other half
after a causal mixing along the sequence, optionally with a single-head "tiny" attention added) and the
output projection. The model-parallel linear layers are plain ``Linear`` layers here; the norm, the
activation and the softmax of the tiny attention run on the kernels of libneox_hotpath.so.
"""
import torch
import torch.nn.functional as F

from .activations import get_activation
from .attention_core import get_fusion_type
from .fused_softmax import FusedScaleMaskSoftmax
from .norms import get_norm


class TinyAttention(torch.nn.Module):
    """Single-head attention of width ``d_attn`` over the block's ``[b, s, 2 * d_ff]`` activation
    (megatron/model/gmlp.py:28-54). The reference multiplies the scores by ``d_attn ** -0.5`` in a pass of its
    own and hands the softmax no scale; with the softmax in fp32 the factor goes into the kernel's scale."""

    def __init__(self, neox_args, d_attn, d_ff, mask_fn):
        super().__init__()
        softmax_in_fp32 = bool(getattr(neox_args, "attention_softmax_in_fp32", False))
        self.scale = d_attn ** -0.5
        self.fold_scale = softmax_in_fp32          # the softmax module only takes a scale when it works in fp32
        self.proj_qkv = torch.nn.Linear(2 * d_ff, 3 * d_attn)
        self.proj_ffn = torch.nn.Linear(d_attn, d_ff)
        self.softmax = FusedScaleMaskSoftmax(
            input_in_fp16=neox_args.precision == "fp16",
            input_in_bf16=neox_args.precision == "bfloat16",
            fusion_type=get_fusion_type(neox_args),
            mask_func=mask_fn,
            softmax_in_fp32=softmax_in_fp32,
            scale=self.scale if self.fold_scale else None,
        )

    def _probabilities(self, queries, keys, attention_mask):
        """``[b, n, d] x [b, m, d] -> [b, n, m]`` attention weights; the softmax module wants a head dimension."""
        scores = torch.bmm(queries, keys.transpose(1, 2))
        if not self.fold_scale:
            scores = scores * self.scale
        n, m = scores.shape[-2:]
        return self.softmax(scores.unsqueeze(1), attention_mask[..., :n, :m]).squeeze(1)

    def forward(self, x, attention_mask):
        queries, keys, values = self.proj_qkv(x).chunk(3, dim=-1)
        mixed = torch.bmm(self._probabilities(queries, keys, attention_mask), values)
        return self.proj_ffn(mixed)


class SpatialGatingUnit(torch.nn.Module):
    """``res * (W_causal . norm(gate) + b [+ tiny attention])`` with ``res, gate`` the two halves of the features
    and ``W`` an ``s x s`` matrix mixing positions, its upper triangle zeroed (megatron/model/gmlp.py:57-94).
    The mixing starts out as the identity on the bias alone: zero weights, unit bias."""

    def __init__(self, neox_args, d_ff, d_attn=None, causal=True, mask_fn=None):
        super().__init__()
        norm_class, eps = get_norm(neox_args)
        self.causal = causal
        self.norm = norm_class(d_ff, eps=eps)
        self.proj = torch.nn.Linear(neox_args.seq_length, neox_args.seq_length)
        with torch.no_grad():
            self.proj.weight.zero_()
            self.proj.bias.fill_(1.0)
        self.use_attn = d_attn is not None
        if self.use_attn:
            assert mask_fn is not None
            self.attn = TinyAttention(neox_args=neox_args, d_attn=d_attn, d_ff=d_ff, mask_fn=mask_fn)

    def _mixing(self, n):
        """Weights ``[n, n]`` and bias ``[n]`` of the mixing along the sequence for ``n`` positions; causal: a
        position only receives from itself and earlier ones."""
        weight, bias = self.proj.weight, self.proj.bias
        if self.causal:
            return torch.tril(weight[:n, :n]), bias[:n]
        return weight, bias

    def forward(self, x, attention_mask):
        batch_first = x.transpose(0, 1)                                   # [s, b, d] -> [b, s, d]
        res, gate = batch_first.chunk(2, dim=-1)
        weight, bias = self._mixing(x.shape[0])
        # positions are mixed as the last dimension of [b, d, s]
        gate = F.linear(self.norm(gate).transpose(1, 2), weight, bias).transpose(1, 2)
        if self.use_attn:
            gate = gate + self.attn(batch_first, attention_mask)
        return (res * gate).transpose(0, 1)                               # -> [s, b, d]


class GMLPBlock(torch.nn.Module):
    """``x -> output_linear(sgu(activation(input_linear(norm(x)))))`` (megatron/model/gmlp.py:97-141); takes and
    returns ``(x, attention_mask)``; ``d_attn`` switches the tiny attention on (the reference's "amlp" layers).

    As in the reference the two projections are created with biases that ``forward`` does not add (its
    linear layers hand the bias back, ``skip_bias_add``, and the block drops it). One setting differs: with
    ``bias_gelu_fusion`` the activation is the fused ``bias_gelu(x, bias)``, which needs the bias and gets the
    input projection's; the reference calls it with one argument and cannot run in that setting."""

    def __init__(self, neox_args, layer_number, ff_mult=4, mask_fn=None, d_attn=None):
        super().__init__()
        self.layer_number = layer_number
        ff_dim = neox_args.hidden_size * ff_mult
        norm, eps = get_norm(neox_args)
        self.norm = norm(neox_args.hidden_size, eps=eps)
        self.input_linear = torch.nn.Linear(neox_args.hidden_size, ff_dim * 2)
        self.activation_func, _ = get_activation(neox_args)
        self.fused_bias_gelu = neox_args.activation == "gelu" and getattr(neox_args, "bias_gelu_fusion", False)
        self.sgu = SpatialGatingUnit(neox_args, ff_dim, d_attn, causal=True, mask_fn=mask_fn)
        self.output_linear = torch.nn.Linear(ff_dim, neox_args.hidden_size)

    def forward(self, args):
        assert len(args) == 2, "GMLPBlock expects 2 arguments"
        x, attention_mask = args
        x = F.linear(self.norm(x), self.input_linear.weight)
        x = self.activation_func(x, self.input_linear.bias) if self.fused_bias_gelu else self.activation_func(x)
        x = self.sgu(x, attention_mask)
        return F.linear(x, self.output_linear.weight), attention_mask
