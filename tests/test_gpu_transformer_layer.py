"""One transformer layer assembled from the fused kernels (megatron/model/transformer_layer.py, the data flow of
ParallelTransformerLayer, megatron/model/transformer.py:962-1321) against the same layer written with plain torch
ops in fp32 on the same parameters, forward and backward.

Tolerance: relative Frobenius error. The layer runs its GEMMs and stores its intermediates in bf16, the reference
runs in fp32, so 2^-6 for the output and 2^-5 for gradients (several bf16 roundings in a row); each kernel on its own
is held to 2 ulp elsewhere."""
import math
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
    base = dict(hidden_size=512, num_attention_heads=8, seq_length=256, precision="bfloat16", pos_emb="rotary",
                rotary_pct=0.25, rotary_emb_base=10000, rope_fusion=True, norm="layernorm", layernorm_epsilon=1e-5,
                rms_norm_epsilon=1e-6, layernorm_fusion=False, rmsnorm_fusion=False, activation="gelu",
                bias_gelu_fusion=True, onnx_safe=False, scaled_upper_triang_masked_softmax_fusion=True,
                scaled_masked_softmax_fusion=False, attention_softmax_in_fp32=True, apply_query_key_layer_scaling=False,
                attention_dropout=0.0, hidden_dropout=0.0, bias_dropout_fusion=True, gpt_j_residual=False,
                gpt_j_tied=False, use_bias_in_mlp=True, use_bias_in_attn_linear=True, intermediate_size=None,
                expansion_factor=None, num_kv_heads=None, sliding_window_width=None)
    base.update(kw)
    return types.SimpleNamespace(**base)


def reference_layer(layer, cfg, x, mask):
    """The same layer in fp32 torch ops, reading the parameters of `layer` (autograd reaches them through .float())."""
    h = cfg.hidden_size
    np_, hn = cfg.num_attention_heads, cfg.hidden_size // cfg.num_attention_heads
    x = x.float()

    def norm(mod, t):
        if cfg.norm == "layernorm":
            return F.layer_norm(t, (h,), mod.weight.float(), mod.bias.float(), cfg.layernorm_epsilon)
        rms = t.norm(2, dim=-1, keepdim=True) * h ** -0.5
        return mod.scale.float() * (t / (rms + cfg.rms_norm_epsilon))

    def lin(mod, t):
        return F.linear(t, mod.weight.float(), None if mod.bias is None else mod.bias.float())

    def attention(t):
        sq, b = t.shape[:2]
        att = layer.attention
        nkv = cfg.num_kv_heads or np_
        if nkv == np_:
            q, k, v = lin(att.query_key_value, t).view(sq, b, np_, 3 * hn).split(hn, dim=-1)
        else:   # [q heads | k heads | v heads]; the k/v heads repeated for the query heads that share them
            q, k, v = lin(att.query_key_value, t).split((np_ * hn, nkv * hn, nkv * hn), dim=-1)
            q = q.view(sq, b, np_, hn)
            k, v = (torch.repeat_interleave(u.view(sq, b, nkv, hn), np_ // nkv, dim=2) for u in (k, v))
        if att.rotary_emb is not None:
            nd = att.rotary_ndims or hn
            cos, sin = att.rotary_emb(t, seq_len=sq)
            cos, sin = cos.float(), sin.float()

            def rot(u):
                r, p = u[..., :nd], u[..., nd:]
                half = torch.cat((-r[..., nd // 2:], r[..., :nd // 2]), dim=-1)
                return torch.cat((r * cos + half * sin, p), dim=-1)

            q, k = rot(q), rot(k)
        q, k, v = (u.permute(1, 2, 0, 3) for u in (q, k, v))
        scores = q @ k.transpose(-1, -2) / math.sqrt(hn)
        if att.core.rpe is not None:
            scores = scores + att.core.rpe(sq, sq).float()
        scores = scores.masked_fill(mask, float("-inf"))
        ctx = (torch.softmax(scores, -1) @ v).permute(2, 0, 1, 3).reshape(sq, b, h)
        return lin(att.dense, ctx)

    def mlp(t):
        u = lin(layer.mlp.linear1, t)
        if cfg.activation == "gelu":
            u = F.gelu(u, approximate="tanh")
        else:  # swiglu
            val, gate = u.chunk(2, dim=-1)
            u = F.silu(gate) * val
        return lin(layer.mlp.linear2, u)

    if cfg.gpt_j_residual:
        return x + attention(norm(layer.input_layernorm, x)) + mlp(norm(layer.post_attention_layernorm, x))
    x = x + attention(norm(layer.input_layernorm, x))
    return x + mlp(norm(layer.post_attention_layernorm, x))


def rel_err(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


@pytest.mark.parametrize("variant", ["pythia", "sequential", "llama", "gqa", "gqa-eager-rope", "rpe", "pythia-2048",
                                     "mistral-2048"])
def test_layer_matches_plain_torch(variant):
    from megatron.model.transformer_layer import TransformerLayer

    cfg = {"pythia": args_for(gpt_j_residual=True),
           "sequential": args_for(rotary_pct=1.0),
           "llama": args_for(norm="rmsnorm", activation="swiglu", rotary_pct=1.0, use_bias_in_mlp=False,
                             use_bias_in_attn_linear=False),
           "gqa": args_for(norm="rmsnorm", activation="swiglu", rotary_pct=1.0, use_bias_in_mlp=False,
                           use_bias_in_attn_linear=False, num_kv_heads=2),
           "gqa-eager-rope": args_for(num_kv_heads=4, rope_fusion=False),
           "rpe": args_for(pos_emb="rpe"),
           # 2048 positions: the attention GEMMs and the softmax work on the blocks below the diagonal only
           "pythia-2048": args_for(gpt_j_residual=True, seq_length=2048),
           "mistral-2048": args_for(norm="rmsnorm", activation="swiglu", rotary_pct=1.0, use_bias_in_mlp=False,
                                    use_bias_in_attn_linear=False, num_kv_heads=2, seq_length=2048,
                                    sliding_window_width=700)}[variant]
    torch.manual_seed(0)
    rpe = None
    if variant == "rpe":   # T5 relative position bias shared by the layers, added inside the softmax kernel
        from megatron.model.positional_embeddings import RelativePositionBias
        rpe = RelativePositionBias(scale=math.sqrt(cfg.hidden_size // cfg.num_attention_heads), causal=True,
                                   num_buckets=32, max_distance=128, heads=cfg.num_attention_heads)
    layer = TransformerLayer(cfg, mask_func, layer_number=3, rpe=rpe, rotary=variant != "rpe").to(DEV)
    with torch.no_grad():   # parameters away from their initial 1 / 0 so that every term matters
        for name, p in layer.named_parameters():
            if p.dim() == 1:
                p.add_(0.1 * torch.randn_like(p))
    layer = layer.to(torch.bfloat16)
    s, b, h = cfg.seq_length, 2, cfg.hidden_size
    x = util.randn((s, b, h), torch.bfloat16, seed=1).to(DEV).requires_grad_(True)
    g = util.randn((s, b, h), torch.bfloat16, seed=2).to(DEV)
    mask = fb.causal_mask(s, DEV, sliding_window_width=getattr(cfg, "sliding_window_width", None))
    if s >= 2048:
        assert layer.attention.core._causal_block(mask, b, cfg.num_attention_heads, s, s, x) == 512
    layer.train()
    out = layer(x, mask)
    assert out.shape == (s, b, h) and out.dtype == torch.bfloat16
    out.backward(g)
    got = {n: p.grad.detach().clone() for n, p in layer.named_parameters()}
    got_dx = x.grad.detach().clone()
    layer.zero_grad()
    xr = x.detach().clone().requires_grad_(True)
    ref = reference_layer(layer, cfg, xr, mask)
    ref.backward(g.float())
    assert rel_err(out, ref) <= 2.0 ** -6
    assert rel_err(got_dx, xr.grad) <= 2.0 ** -5
    for n, p in layer.named_parameters():
        assert p.grad is not None and n in got, n
        assert rel_err(got[n], p.grad) <= 2.0 ** -5, n
    # evaluation mode takes the same path when every dropout probability is zero
    layer.eval()
    with torch.no_grad():
        assert torch.equal(layer(x.detach(), mask), out.detach())


def test_layer_with_dropout_trains_and_is_repeatable():
    from megatron.model.transformer_layer import TransformerLayer

    cfg = args_for(gpt_j_residual=True, attention_dropout=0.1, hidden_dropout=0.1)
    torch.manual_seed(0)
    layer = TransformerLayer(cfg, mask_func, layer_number=1, rotary=True).to(DEV).to(torch.bfloat16)
    s, b, h = 256, 2, cfg.hidden_size
    x = util.randn((s, b, h), torch.bfloat16, seed=1).to(DEV)
    mask = fb.causal_mask(s, DEV)
    layer.train()
    torch.manual_seed(7)
    a = layer(x, mask)
    torch.manual_seed(7)
    again = layer(x, mask)
    torch.manual_seed(8)
    other = layer(x, mask)
    layer.eval()
    quiet = layer(x, mask)
    assert torch.equal(a, again) and not torch.equal(a, other) and not torch.equal(a, quiet)
    assert rel_err(a, quiet) < 0.5
    layer.train()
    xg = x.clone().requires_grad_(True)
    layer(xg, mask).float().square().mean().backward()
    assert torch.isfinite(xg.grad.float()).all() and all(torch.isfinite(p.grad.float()).all() for p in layer.parameters())


def test_layer_under_activation_checkpointing_reproduces_its_dropout_masks():
    """With activation checkpointing (GPT-NeoX's `checkpoint-activations`) the forward runs a second time in the
    backward; the dropout seeds come from torch's CPU generator, whose state checkpointing restores, so the recomputed
    masks are the ones of the first pass and the gradients equal those of a run without checkpointing."""
    from torch.utils.checkpoint import checkpoint

    from megatron.model.transformer_layer import TransformerLayer

    cfg = args_for(gpt_j_residual=True, attention_dropout=0.1, hidden_dropout=0.1)
    torch.manual_seed(0)
    layer = TransformerLayer(cfg, mask_func, layer_number=1, rotary=True).to(DEV).to(torch.bfloat16).train()
    s, b, h = 256, 2, cfg.hidden_size
    x = util.randn((s, b, h), torch.bfloat16, seed=1).to(DEV)
    g = util.randn((s, b, h), torch.bfloat16, seed=2).to(DEV)
    mask = fb.causal_mask(s, DEV)

    def run(use_checkpoint):
        layer.zero_grad(set_to_none=True)
        xg = x.clone().requires_grad_(True)
        torch.manual_seed(21)
        out = checkpoint(layer, xg, mask, use_reentrant=False) if use_checkpoint else layer(xg, mask)
        out.backward(g)
        return out.detach(), xg.grad, {n: p.grad.clone() for n, p in layer.named_parameters()}

    out_a, dx_a, grads_a = run(False)
    out_b, dx_b, grads_b = run(True)
    assert torch.equal(out_a, out_b) and torch.equal(dx_a, dx_b)
    for n in grads_a:
        assert torch.equal(grads_a[n], grads_b[n]), n


@pytest.mark.parametrize("variant", ["pythia", "gqa", "eager-rope"])
def test_incremental_decoding_with_cached_keys_equals_the_full_pass(variant):
    """use_cache (megatron/model/transformer.py:916-935, 1219-1225): feeding the sequence in pieces, each call
    continuing after the cached keys and values, gives the hidden states of one pass over the whole sequence.
    Pieces of 64 (masked kernel on a rectangular score matrix), 3 and 1 positions (torch branch of the softmax)."""
    from megatron.model.transformer_layer import TransformerLayer

    cfg = {"pythia": args_for(gpt_j_residual=True),
           "gqa": args_for(norm="rmsnorm", activation="swiglu", rotary_pct=1.0, use_bias_in_mlp=False,
                           use_bias_in_attn_linear=False, num_kv_heads=2),
           "eager-rope": args_for(rope_fusion=False)}[variant]
    torch.manual_seed(0)
    layer = TransformerLayer(cfg, mask_func, layer_number=1, rotary=True, use_cache=True).to(DEV).to(torch.bfloat16).eval()
    s, b, h = 136, 4, cfg.hidden_size
    x = util.randn((s, b, h), torch.bfloat16, seed=1).to(DEV)
    mask = fb.causal_mask(s, DEV)
    nkv = cfg.num_kv_heads or cfg.num_attention_heads
    with torch.no_grad():
        full = layer(x, mask)
        assert layer.layer_past.shape == (2, s, b, nkv, h // cfg.num_attention_heads)
        layer.layer_past = None
        pieces, start = [], 0
        for n in (64, 64, 3, 1, 4):
            rows = mask[..., start:start + n, :start + n]
            pieces.append(layer(x[start:start + n], rows))
            start += n
            assert layer.layer_past.shape[1] == start
        assert start == s
    got = torch.cat(pieces, dim=0)
    # the same arithmetic per position up to the order of the GEMMs' sums
    assert rel_err(got, full) <= 2.0 ** -7
    assert (got.float() - full.float()).abs().max() <= 2.0 ** -4 * full.float().abs().max()
