"""The fused path inside the computation that surrounds it in GPT-NeoX
(ParallelSelfAttention, megatron/model/transformer.py:841-959): fused QKV
projection -> rotary on q, k (partial rotary) -> baddbmm scores -> scale-mask-softmax
-> probabilities @ V, forward and backward, once with the fused kernels and once
with the reference's unfused torch operations. The two must agree to the
accuracy of the storage dtype (they differ only by the <= 1 ulp differences of
the softmax and by torch's own matmul rounding, which is identical on both sides)."""
import math

import pytest
import torch

import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"


def attention(qkv, rotary, softmax_module, mask, fused_rope, rot_dim, hn, norm_factor):
    from megatron.model.fused_rope import fused_apply_rotary_pos_emb_cached
    from megatron.model.positional_embeddings import apply_rotary_pos_emb_torch

    sq, b, np_, _ = qkv.shape
    q, k, v = torch.split(qkv, hn, dim=3)  # non-contiguous views, as in NeoX
    cos, sin = rotary(v, seq_len=sq)
    if rot_dim < hn:
        q_rot, q_pass = q[..., :rot_dim], q[..., rot_dim:]
        k_rot, k_pass = k[..., :rot_dim], k[..., rot_dim:]
    else:
        q_rot, k_rot = q, k
    if fused_rope:
        q_rot = fused_apply_rotary_pos_emb_cached(q_rot, cos, sin)
        k_rot = fused_apply_rotary_pos_emb_cached(k_rot, cos, sin)
    else:
        q_rot, k_rot = apply_rotary_pos_emb_torch(q_rot, k_rot, cos, sin, offset=0)
    if rot_dim < hn:
        q = torch.cat((q_rot, q_pass), dim=-1)
        k = torch.cat((k_rot, k_pass), dim=-1)
    else:
        q, k = q_rot, k_rot
    q2 = q.reshape(sq, b * np_, hn)
    k2 = k.reshape(sq, b * np_, hn)
    scores = torch.baddbmm(
        torch.empty(b * np_, sq, sq, dtype=q.dtype, device=q.device),
        q2.transpose(0, 1), k2.transpose(0, 1).transpose(1, 2), beta=0.0, alpha=1.0 / norm_factor)
    probs = softmax_module(scores.view(b, np_, sq, sq), mask)
    v2 = v.reshape(sq, b * np_, hn)
    ctx = torch.bmm(probs.view(b * np_, sq, sq), v2.transpose(0, 1))
    return ctx.view(b, np_, sq, hn), probs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("rotary_pct", [1.0, 0.25])
def test_attention_block_fused_vs_unfused(dtype, rotary_pct):
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T
    from megatron.model.positional_embeddings import RotaryEmbedding

    sq, b, np_, hn = 256, 2, 4, 64
    rot_dim = int(hn * rotary_pct)
    norm_factor = math.sqrt(hn)
    qkv0 = util.randn((sq, b, np_, 3 * hn), dtype, seed=1, std=1.0)
    gctx = util.randn((b, np_, sq, hn), dtype, seed=2).to(DEV)
    rotary = RotaryEmbedding(rot_dim, sq, precision=dtype)
    mask = fb.causal_mask(sq, DEV)
    results = {}
    for name, fusion, fused_rope in (("fused", T.upper_triang, True), ("unfused", T.none, False)):
        sm = FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, fusion,
                                   fb.fill_masked_with_dtype_min, True, None)
        qkv = qkv0.to(DEV).requires_grad_(True)
        ctx, probs = attention(qkv, rotary, sm, mask, fused_rope, rot_dim, hn, norm_factor)
        ctx.backward(gctx)
        results[name] = (ctx.detach().float().cpu(), probs.detach().cpu(), qkv.grad.float().cpu())
    cf, pf, gf = results["fused"]
    cu, pu, gu = results["unfused"]
    # rotary is bit-exact, so the scores are identical and the probabilities differ by the softmax only
    util.assert_ulp_close(pf, pu, 2, "probabilities")
    eps = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-11
    assert (cf - cu).abs().max().item() <= 8 * eps * cu.abs().max().item()
    # gradients w.r.t. the fused projection: the fused backward starts from rounded probabilities,
    # autograd through the torch path from fp32 ones
    assert (gf - gu).abs().max().item() <= 16 * eps * gu.abs().max().item()
    rel = (gf - gu).norm().item() / gu.norm().item()
    assert rel < 4 * eps, rel
