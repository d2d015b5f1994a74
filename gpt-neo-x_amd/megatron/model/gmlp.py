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
        self.proj_qkv = torch.nn.Linear(d_ff * 2, 3 * d_attn)
        self.proj_ffn = torch.nn.Linear(d_attn, d_ff)
        self.scale = d_attn ** -0.5
        in_fp32 = getattr(neox_args, "attention_softmax_in_fp32", False)
        self.fold_scale = bool(in_fp32)
        self.softmax = FusedScaleMaskSoftmax(
            input_in_fp16=neox_args.precision == "fp16", input_in_bf16=neox_args.precision == "bfloat16",
            fusion_type=get_fusion_type(neox_args), mask_func=mask_fn, softmax_in_fp32=in_fp32,
            scale=self.scale if self.fold_scale else None)

    def forward(self, x, attention_mask):
        q, k, v = torch.chunk(self.proj_qkv(x), 3, dim=-1)
        scores = torch.bmm(q, k.transpose(1, 2)).unsqueeze(1)          # [b, 1, n, m]
        if not self.fold_scale:
            scores = scores * self.scale
        mask = attention_mask[..., :scores.size(-2), :scores.size(-1)]
        probs = self.softmax(scores, mask).squeeze(1)
        return self.proj_ffn(torch.bmm(probs, v))


class SpatialGatingUnit(torch.nn.Module):
    """``res * (W_causal . norm(gate) + b [+ tiny attention])`` with ``res, gate`` the two halves of the features
    and ``W`` an ``s x s`` matrix mixing positions, its upper triangle zeroed (megatron/model/gmlp.py:57-94)."""

    def __init__(self, neox_args, d_ff, d_attn=None, causal=True, mask_fn=None):
        super().__init__()
        self.causal = causal
        self.use_attn = d_attn is not None
        norm, eps = get_norm(neox_args)
        self.norm = norm(d_ff, eps=eps)
        self.proj = torch.nn.Linear(neox_args.seq_length, neox_args.seq_length)
        if self.use_attn:
            assert mask_fn is not None
            self.attn = TinyAttention(neox_args, d_attn, d_ff, mask_fn)
        torch.nn.init.zeros_(self.proj.weight)
        torch.nn.init.constant_(self.proj.bias, 1.0)

    def forward(self, x, attention_mask):
        n = x.shape[0]
        x = x.transpose(0, 1)                                            # [s, b, d] -> [b, s, d]
        res, gate = x.chunk(2, dim=-1)
        gate = self.norm(gate)
        weight, bias = self.proj.weight, self.proj.bias
        if self.causal:
            weight, bias = torch.tril(weight[:n, :n]), bias[:n]
        # mixing along the sequence: [b, d, s] x W^T + b
        gate = F.linear(gate.transpose(1, 2), weight, bias).transpose(1, 2)
        if self.use_attn:
            gate = gate + self.attn(x, attention_mask)
        return (gate * res).transpose(0, 1)                              # -> [s, b, d]


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
