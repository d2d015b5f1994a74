"""The gMLP / aMLP block (megatron/model/gmlp.py:28-141 of the reference), the second caller of the fused softmax,
assembled from the fused norm, activation and softmax kernels, against the same block in fp32 torch ops on the same
parameters; forward and backward. Tolerance: relative Frobenius error, as for the transformer layer (bf16 GEMMs and
intermediates against fp32)."""
import types

import pytest
import torch
import torch.nn.functional as F

import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"


def mask_func(scores, mask):
    return fb.fill_masked_with_dtype_min(scores, mask)


def args_for(**kw):
    base = dict(hidden_size=256, seq_length=128, precision="bfloat16", norm="layernorm", layernorm_epsilon=1e-5,
                rms_norm_epsilon=1e-6, layernorm_fusion=False, rmsnorm_fusion=False, activation="gelu",
                bias_gelu_fusion=False, onnx_safe=False, scaled_upper_triang_masked_softmax_fusion=True,
                scaled_masked_softmax_fusion=False, attention_softmax_in_fp32=True)
    base.update(kw)
    return types.SimpleNamespace(**base)


def reference_block(block, cfg, x, mask):
    def norm(mod, t):
        return F.layer_norm(t, (t.size(-1),), mod.weight.float(), mod.bias.float(), cfg.layernorm_epsilon)

    x = norm(block.norm, x.float())
    x = F.linear(x, block.input_linear.weight.float())
    if block.fused_bias_gelu:
        x = F.gelu(x + block.input_linear.bias.float(), approximate="tanh")
    else:
        x = F.gelu(x)
    sgu = block.sgu
    x = x.transpose(0, 1)
    res, gate = x.chunk(2, dim=-1)
    gate = norm(sgu.norm, gate)
    n = x.size(1)
    w = torch.tril(sgu.proj.weight.float()[:n, :n])
    gate = torch.einsum("nm,bmd->bnd", w, gate) + sgu.proj.bias.float()[:n, None]
    if sgu.use_attn:
        att = sgu.attn
        q, k, v = F.linear(x, att.proj_qkv.weight.float(), att.proj_qkv.bias.float()).chunk(3, dim=-1)
        scores = (q @ k.transpose(1, 2) * att.scale).masked_fill(mask[0], float("-inf"))
        gate = gate + F.linear(torch.softmax(scores, -1) @ v, att.proj_ffn.weight.float(), att.proj_ffn.bias.float())
    return F.linear((gate * res).transpose(0, 1), block.output_linear.weight.float())


def rel_err(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


@pytest.mark.parametrize("variant", ["gmlp", "amlp", "amlp-fused-gelu"])
def test_gmlp_block_matches_plain_torch(variant):
    from megatron.model.gmlp import GMLPBlock

    cfg = args_for(bias_gelu_fusion=variant == "amlp-fused-gelu")
    d_attn = None if variant == "gmlp" else 64
    torch.manual_seed(0)
    block = GMLPBlock(cfg, layer_number=0, ff_mult=2, mask_fn=mask_func, d_attn=d_attn).to(DEV)
    with torch.no_grad():
        block.sgu.proj.weight.normal_(0, 0.05)   # the zero initial mixing matrix would hide the causal part
        for p in block.parameters():
            if p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
    block = block.to(torch.bfloat16)
    s, b, h = cfg.seq_length, 4, cfg.hidden_size
    x = util.randn((s, b, h), torch.bfloat16, seed=1).to(DEV).requires_grad_(True)
    g = util.randn((s, b, h), torch.bfloat16, seed=2).to(DEV)
    mask = fb.causal_mask(s, DEV)
    out, same_mask = block((x, mask))
    assert same_mask is mask and out.shape == (s, b, h) and out.dtype == torch.bfloat16
    if d_attn is not None:   # the tiny attention's scores [b, 1, s, s] take the fused causal kernel
        assert block.sgu.attn.softmax.is_kernel_available(mask, b, 1, s, s)
    out.backward(g)
    got = {n: p.grad.detach().clone() for n, p in block.named_parameters() if p.grad is not None}
    got_dx = x.grad.detach().clone()
    block.zero_grad()
    xr = x.detach().clone().requires_grad_(True)
    ref = reference_block(block, cfg, xr, mask)
    ref.backward(g.float())
    assert rel_err(out, ref) <= 2.0 ** -6
    assert rel_err(got_dx, xr.grad) <= 2.0 ** -5
    unused = {"input_linear.bias", "output_linear.bias"} - ({"input_linear.bias"} if block.fused_bias_gelu else set())
    for n, p in block.named_parameters():
        if n in unused:
            assert p.grad is None and n not in got   # created, never added: as in the reference
            continue
        assert rel_err(got[n], p.grad) <= 2.0 ** -5, n
    # causality: the output at position t does not depend on later inputs
    with torch.no_grad():
        x2 = x.detach().clone()
        x2[s // 2:] += 1.0
        out2, _ = block((x2, mask))
        assert torch.equal(out2[:s // 2], out.detach()[:s // 2])
