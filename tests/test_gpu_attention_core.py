"""The caller of the fused softmax on the GPU: CoreAttention (the score -> probability ->
context part of ParallelSelfAttention.attention, megatron/model/transformer.py:526-625) against
textbook attention evaluated in fp32 with torch ops, forward and backward.

Tolerance: the two GEMMs run in the 16-bit storage type, so results are compared by relative
Frobenius error (2^-7 for bf16, 2^-9 for fp16), not by units in the last place; the softmax
kernel itself is held to 2 ulp in the other GPU tests."""
import math

import pytest
import torch

import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"


def mask_func(scores, mask):
    return fb.fill_masked_with_dtype_min(scores, mask)


def textbook(q, k, v, mask, extra=None):
    """softmax(q k^T / sqrt(hn) + extra, masked) v in fp32; q [sq,b,np,hn] -> [b,np,sq,hn]."""
    q, k, v = (t.float().permute(1, 2, 0, 3) for t in (q, k, v))
    scores = q @ k.transpose(-1, -2) / math.sqrt(q.size(-1))
    if extra is not None:
        scores = scores + extra
    scores = scores.masked_fill(mask, float("-inf"))
    return torch.softmax(scores, dim=-1) @ v


def rel_err(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm()).item()


def qkv(dtype, sq, b, np_, hn, seed):
    return [util.randn((sq, b, np_, hn), dtype, seed=seed + i).to(DEV).requires_grad_(True) for i in range(3)]


@pytest.mark.parametrize("layer_scaling", [False, True], ids=["plain", "qk-layer-scaling"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_causal_attention_matches_textbook(dtype, layer_scaling):
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    sq, b, np_, hn = 512, 2, 4, 64
    lim = 2.0 ** (-7 if dtype == torch.bfloat16 else -9)
    core = CoreAttention(hn, 7, dtype == torch.float16, dtype == torch.bfloat16, T.upper_triang, mask_func,
                         attention_softmax_in_fp32=True, apply_query_key_layer_scaling=layer_scaling)
    assert core.norm_factor == math.sqrt(hn) * (7 if layer_scaling else 1)
    if dtype == torch.float16:   # the reference's split: 1 / norm_factor in the GEMM, coeff in the softmax
        assert not core.fold_scale and core.gemm_alpha == 1 / core.norm_factor
        assert core.scale_mask_softmax.scale == (7 if layer_scaling else None)
    else:                        # both factors in the softmax kernel's fp32 scale
        assert core.fold_scale and core.gemm_alpha == 1.0
        assert core.scale_mask_softmax.scale == pytest.approx(1 / math.sqrt(hn))
    q, k, v = qkv(dtype, sq, b, np_, hn, 1)
    mask = fb.causal_mask(sq, DEV)
    assert core.scale_mask_softmax.is_kernel_available(mask, b, np_, sq, sq)
    out = core(q, k, v, mask)
    assert out.shape == (b, np_, sq, hn) and out.dtype == dtype
    g = util.randn((b, np_, sq, hn), dtype, seed=9).to(DEV)
    out.backward(g)
    qr, kr, vr = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    ref = textbook(qr, kr, vr, mask)
    ref.backward(g.float())
    assert rel_err(out, ref) <= lim
    for got, want in ((q.grad, qr.grad), (k.grad, kr.grad), (v.grad, vr.grad)):
        assert rel_err(got, want) <= 2 * lim
    # folding the GEMM's factor into the softmax scale changes nothing beyond bf16 rounding of the scores
    if dtype == torch.bfloat16:
        split = CoreAttention(hn, 7, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True,
                              apply_query_key_layer_scaling=layer_scaling, fold_scale=False)
        assert not split.fold_scale and split.scale_mask_softmax.scale == (7 if layer_scaling else None)
        assert rel_err(split(q.detach(), k.detach(), v.detach(), mask), ref) <= lim
    # the fused and the torch branch of the softmax module agree inside the caller
    plain = CoreAttention(hn, 7, dtype == torch.float16, dtype == torch.bfloat16, T.none, mask_func,
                          attention_softmax_in_fp32=True, apply_query_key_layer_scaling=layer_scaling)
    assert rel_err(plain(q.detach(), k.detach(), v.detach(), mask), out) <= lim


def test_padding_mask_alibi_window_and_rpe_inside_the_caller():
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T
    from megatron.model.positional_embeddings import AliBi

    dtype, sq, b, np_, hn = torch.bfloat16, 256, 4, 4, 64
    lim = 2.0 ** -7
    q, k, v = qkv(dtype, sq, b, np_, hn, 11)
    pos = torch.arange(sq, device=DEV)
    causal = fb.causal_mask(sq, DEV)

    # padding mask through the general kernel
    lengths = torch.tensor([256, 200, 64, 1], device=DEV)
    pad = (pos.view(1, 1, 1, sq) >= lengths.view(b, 1, 1, 1)).expand(b, 1, sq, sq).contiguous()
    core = CoreAttention(hn, 1, False, True, T.general, mask_func, attention_softmax_in_fp32=True)
    assert rel_err(core(q, k, v, pad), textbook(q, k, v, pad)) <= lim

    # the same padding by key lengths on the causal kernel
    core = CoreAttention(hn, 1, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True)
    both = causal | pad
    assert rel_err(core(q, k, v, causal, key_lengths=lengths.int()), textbook(q, k, v, both)) <= lim

    # AliBi inside the kernel
    slopes = AliBi(np_, 1, 0).slopes
    core = CoreAttention(hn, 1, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True, alibi_slopes=slopes)
    dist = -(pos.view(sq, 1) - pos.view(1, sq)).clamp(min=0).float()
    extra = dist.view(1, 1, sq, sq) * slopes.to(DEV).float().view(1, np_, 1, 1)
    assert rel_err(core(q, k, v, causal), textbook(q, k, v, causal, extra)) <= lim

    # sliding window of 32 keys
    window = causal | (pos.view(1, sq) < pos.view(sq, 1) - 32).view(1, 1, sq, sq)
    core = CoreAttention(hn, 1, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True, sliding_window_width=32)
    assert rel_err(core(q, k, v, window), textbook(q, k, v, window)) <= lim

    # relative position bias handed to the kernel as a tensor
    table = util.randn((1, np_, sq, sq), dtype, seed=3, std=0.5).to(DEV)
    core = CoreAttention(hn, 1, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True,
                         rpe=lambda a, c: table[..., :a, :c])
    assert rel_err(core(q, k, v, causal), textbook(q, k, v, causal, table.float())) <= lim


def test_attention_dropout_inside_the_caller():
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    dtype, sq, b, np_, hn = torch.bfloat16, 256, 2, 4, 64
    q, k, v = (t.detach() for t in qkv(dtype, sq, b, np_, hn, 21))
    mask = fb.causal_mask(sq, DEV)
    core = CoreAttention(hn, 1, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True, attention_dropout=0.2)
    core.eval()
    quiet = core(q, k, v, mask)
    assert rel_err(quiet, textbook(q, k, v, mask)) <= 2.0 ** -7
    core.train()
    torch.manual_seed(5)
    a = core(q, k, v, mask)
    torch.manual_seed(5)
    again = core(q, k, v, mask)
    torch.manual_seed(6)
    other = core(q, k, v, mask)
    assert torch.equal(a, again) and not torch.equal(a, other) and not torch.equal(a, quiet)
    # dropout keeps the expectation: averaged over many masks the result approaches the plain one
    acc = torch.zeros_like(quiet, dtype=torch.float32)
    for i in range(64):
        torch.manual_seed(100 + i)
        acc += core(q, k, v, mask).float()
    assert rel_err(acc / 64, quiet) <= 0.12


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("rotary_ndims", [None, 32], ids=["full", "partial"])
def test_rotary_call_site(dtype, rotary_ndims):
    """apply_rotary_to_query_key (the rotary block of ParallelSelfAttention.forward, transformer.py:877-914) on q and k
    sliced from one fused projection output: the single-launch path, the reference's statement-by-statement fused
    path and the eager path agree bit for bit; with cached keys the single launch follows the eager path (which
    honours the offset), the reference's fused branch does not."""
    from megatron.model.attention_core import apply_rotary_to_query_key
    from megatron.model.positional_embeddings import RotaryEmbedding

    sq, b, np_, hn = 96, 2, 4, 128
    qkv_out = util.randn((sq, b, np_, 3 * hn), dtype, seed=4).to(DEV)
    q, k = qkv_out[..., :hn], qkv_out[..., hn:2 * hn]
    emb = RotaryEmbedding(rotary_ndims or hn, 256, base=10000, precision=dtype)
    bf16 = dtype == torch.bfloat16

    def run(**kw):
        return apply_rotary_to_query_key(q, k, emb, rotary_ndims=rotary_ndims, bf16=bf16, **kw)

    one = run(rope_fusion=True, one_launch=True)
    two = run(rope_fusion=True, one_launch=False)
    eager = run(rope_fusion=False)
    for got in (one, two):
        for a, e in zip(got, eager):
            assert a.shape == (sq, b, np_, hn) and a.is_contiguous()
            assert torch.equal(util.raw_bits(a), util.raw_bits(e))
    # decoding: 40 cached positions
    past = torch.zeros((2, 40, b, np_, hn), dtype=dtype, device=DEV)
    one = run(rope_fusion=True, one_launch=True, layer_past=past)
    eager = run(rope_fusion=False, layer_past=past)
    ref_style = run(rope_fusion=True, one_launch=False, layer_past=past)
    for a, e, r, plain in zip(one, eager, ref_style, two):
        assert torch.equal(util.raw_bits(a), util.raw_bits(e))
        assert torch.equal(util.raw_bits(r), util.raw_bits(plain))     # positions 0..sq-1 whatever the cache holds
        assert not torch.equal(util.raw_bits(a), util.raw_bits(r))
    # gradients flow through both fused paths and agree
    qa = q.detach().clone().requires_grad_(True)
    ka = k.detach().clone().requires_grad_(True)
    outs = apply_rotary_to_query_key(qa, ka, emb, rotary_ndims=rotary_ndims, rope_fusion=True, one_launch=True)
    gq, gk = util.randn((sq, b, np_, hn), dtype, seed=7).to(DEV), util.randn((sq, b, np_, hn), dtype, seed=8).to(DEV)
    torch.autograd.backward(outs, (gq, gk))
    qb = q.detach().clone().requires_grad_(True)
    kb = k.detach().clone().requires_grad_(True)
    outs = apply_rotary_to_query_key(qb, kb, emb, rotary_ndims=rotary_ndims, rope_fusion=True, one_launch=False)
    torch.autograd.backward(outs, (gq, gk))
    assert torch.equal(util.raw_bits(qa.grad), util.raw_bits(qb.grad)) and torch.equal(util.raw_bits(ka.grad), util.raw_bits(kb.grad))


@pytest.mark.parametrize("rotary_ndims", [None, 32], ids=["full", "partial"])
def test_split_and_rotate_matches_split_then_rotate(rotary_ndims):
    """split_qkv_and_rotate against torch.split followed by apply_rotary_to_query_key: same results, and the same
    gradient for the projection output although it is assembled without a concatenation. The key gradient is fed
    in the layout the score GEMM's backward produces (contiguous along the sequence)."""
    from megatron.model.attention_core import apply_rotary_to_query_key, split_qkv_and_rotate
    from megatron.model.positional_embeddings import RotaryEmbedding

    dtype, sq, b, np_, hn = torch.bfloat16, 128, 2, 4, 128
    emb = RotaryEmbedding(rotary_ndims or hn, 256, base=10000, precision=dtype)
    base = util.randn((sq, b, np_, 3 * hn), dtype, seed=4).to(DEV)
    ma = base.clone().requires_grad_(True)
    mb = base.clone().requires_grad_(True)
    qa, ka, va = split_qkv_and_rotate(ma, emb)
    q0, k0, vb = torch.split(mb, hn, dim=-1)
    qb, kb = apply_rotary_to_query_key(q0, k0, emb, rotary_ndims=rotary_ndims, rope_fusion=True, one_launch=True)
    for a, e in ((qa, qb), (ka, kb), (va, vb)):
        assert a.shape == e.shape and torch.equal(util.raw_bits(a), util.raw_bits(e))
    gq = util.randn((sq, b, np_, hn), dtype, seed=5).to(DEV)
    gk = util.randn((b, np_, hn, sq), dtype, seed=6).to(DEV).permute(3, 0, 1, 2)   # [sq, b, np, hn], sequence-major
    gv = util.randn((sq, b, np_, hn), dtype, seed=7).to(DEV)
    torch.autograd.backward((qa, ka, va), (gq, gk, gv))
    torch.autograd.backward((qb, kb, vb), (gq, gk, gv))
    assert torch.equal(util.raw_bits(ma.grad), util.raw_bits(mb.grad))
    # only part of the outputs used
    mc = base.clone().requires_grad_(True)
    qc, kc, vc = split_qkv_and_rotate(mc, emb)
    qc.backward(gq)
    assert torch.equal(util.raw_bits(mc.grad[..., :hn]), util.raw_bits(ma.grad[..., :hn]))
    assert mc.grad[..., hn:].abs().max().item() == 0
    # with cached keys the rotation starts at the position after them
    past = torch.zeros((2, 40, b, np_, hn), dtype=dtype, device=DEV)
    qd, kd, _ = split_qkv_and_rotate(base, emb, layer_past=past)
    qe, ke = apply_rotary_to_query_key(base[..., :hn], base[..., hn:2 * hn], emb, rotary_ndims=rotary_ndims,
                                       rope_fusion=False, bf16=True, layer_past=past)
    assert torch.equal(util.raw_bits(qd), util.raw_bits(qe)) and torch.equal(util.raw_bits(kd), util.raw_bits(ke))


def test_merged_heads_output_equals_the_permuted_context():
    """CoreAttention(..., merged_heads=True) returns permute(2, 0, 1, 3) of the default result, reshaped to
    [sq, b, np * hn] (megatron/model/transformer.py:941-947), bit for bit, with the same gradients."""
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    dtype, sq, b, np_, hn = torch.bfloat16, 256, 2, 4, 64
    core = CoreAttention(hn, 1, False, True, T.upper_triang, mask_func, attention_softmax_in_fp32=True)
    mask = fb.causal_mask(sq, DEV)
    qa, ka, va = qkv(dtype, sq, b, np_, hn, 31)
    qb, kb, vb = (t.detach().clone().requires_grad_(True) for t in (qa, ka, va))
    merged = core(qa, ka, va, mask, merged_heads=True)
    plain = core(qb, kb, vb, mask).permute(2, 0, 1, 3).contiguous().view(sq, b, np_ * hn)
    assert merged.shape == (sq, b, np_ * hn) and merged.is_contiguous()
    assert torch.equal(util.raw_bits(merged), util.raw_bits(plain))
    g = util.randn((sq, b, np_ * hn), dtype, seed=5).to(DEV)
    merged.backward(g)
    plain.backward(g)
    for a, e in ((qa, qb), (ka, kb), (va, vb)):
        assert torch.equal(util.raw_bits(a.grad), util.raw_bits(e.grad))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("merged", [False, True], ids=["bnsh", "merged"])
def test_grouped_query_attention_equals_attention_with_repeated_heads(dtype, merged):
    """k and v with fewer heads than q: the grouped GEMMs against what the reference does, repeat_interleave of
    the k/v heads (gqa_project, megatron/model/transformer.py:820-837) followed by ordinary attention; textbook
    fp32 attention on the repeated heads as the arbiter. The gradients of k and v are the sums over the query heads
    that share them."""
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    sq, b, np_, nkv, hn = 256, 2, 8, 2, 64
    lim = 2.0 ** (-7 if dtype == torch.bfloat16 else -9)
    core = CoreAttention(hn, 1, dtype == torch.float16, dtype == torch.bfloat16, T.upper_triang, mask_func,
                         attention_softmax_in_fp32=True)
    mask = fb.causal_mask(sq, DEV)
    q = util.randn((sq, b, np_, hn), dtype, seed=41).to(DEV).requires_grad_(True)
    k = util.randn((sq, b, nkv, hn), dtype, seed=42).to(DEV).requires_grad_(True)
    v = util.randn((sq, b, nkv, hn), dtype, seed=43).to(DEV).requires_grad_(True)
    out = core(q, k, v, mask, merged_heads=merged)
    shape = (sq, b, np_ * hn) if merged else (b, np_, sq, hn)
    assert out.shape == shape and out.dtype == dtype
    g = util.randn(shape, dtype, seed=44).to(DEV)
    out.backward(g)

    def repeated(t):
        return torch.repeat_interleave(t, np_ // nkv, dim=2)

    # the reference's way through the same module
    q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    out2 = core(q2, repeated(k2), repeated(v2), mask, merged_heads=merged)
    out2.backward(g)
    # textbook fp32
    q3, k3, v3 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    ref = textbook(q3, repeated(k3), repeated(v3), mask)
    if merged:
        ref = ref.permute(2, 0, 1, 3).reshape(shape)
    ref.backward(g.float())
    assert rel_err(out, ref) <= lim and rel_err(out2, ref) <= lim
    for got, same, want in ((q.grad, q2.grad, q3.grad), (k.grad, k2.grad, k3.grad), (v.grad, v2.grad, v3.grad)):
        assert got.shape == want.shape
        assert rel_err(got, want) <= 2 * lim
        # at least as close to the fp32 result as the repeat-and-reduce route
        assert rel_err(got, want) <= 1.5 * rel_err(same, want) + 1e-6
    # probabilities are identical whichever way the scores were formed up to the GEMM's own rounding
    assert rel_err(out, out2) <= lim


def test_split_gqa_and_rotate_matches_split_then_rotate():
    """split_gqa_and_rotate against torch.split with the sizes of gqa_project followed by the rotary call site:
    same q, k, v and the same gradient for the projection output; q and k come back head-major."""
    from megatron.model.attention_core import apply_rotary_to_query_key, split_gqa_and_rotate
    from megatron.model.positional_embeddings import RotaryEmbedding

    dtype, sq, b, np_, nkv, hn = torch.bfloat16, 128, 2, 8, 2, 128
    emb = RotaryEmbedding(hn, 256, base=10000, precision=dtype)
    base = util.randn((sq, b, (np_ + 2 * nkv) * hn), dtype, seed=4).to(DEV)
    ma = base.clone().requires_grad_(True)
    mb = base.clone().requires_grad_(True)
    qa, ka, va = split_gqa_and_rotate(ma, emb, np_, nkv)
    assert qa.shape == (sq, b, np_, hn) and ka.shape == (sq, b, nkv, hn) and va.shape == (sq, b, nkv, hn)
    assert qa.permute(1, 2, 0, 3).is_contiguous() and ka.permute(1, 2, 0, 3).is_contiguous()
    q0, k0, v0 = torch.split(mb, (np_ * hn, nkv * hn, nkv * hn), dim=-1)
    q0, k0, vb = q0.view(sq, b, np_, hn), k0.view(sq, b, nkv, hn), v0.view(sq, b, nkv, hn)
    qb, kb = apply_rotary_to_query_key(q0, k0, emb, rope_fusion=True, one_launch=True)
    for a, e in ((qa, qb), (ka, kb), (va, vb)):
        assert a.shape == e.shape and torch.equal(util.raw_bits(a), util.raw_bits(e))
    # gradients in the layouts the grouped GEMMs hand back: q head-major, k contiguous along the sequence
    gq = util.randn((b, np_, sq, hn), dtype, seed=5).to(DEV).permute(2, 0, 1, 3)
    gk = util.randn((b, nkv, hn, sq), dtype, seed=6).to(DEV).permute(3, 0, 1, 2)
    gv = util.randn((b, nkv, sq, hn), dtype, seed=7).to(DEV).permute(2, 0, 1, 3)
    torch.autograd.backward((qa, ka, va), (gq, gk, gv))
    torch.autograd.backward((qb, kb, vb), (gq, gk, gv))
    assert torch.equal(util.raw_bits(ma.grad), util.raw_bits(mb.grad))
    # only the keys used
    mc = base.clone().requires_grad_(True)
    _, kc, _ = split_gqa_and_rotate(mc, emb, np_, nkv)
    kc.backward(gk)
    lo, hi = np_ * hn, (np_ + nkv) * hn
    assert torch.equal(util.raw_bits(mc.grad[..., lo:hi]), util.raw_bits(ma.grad[..., lo:hi]))
    assert mc.grad[..., :lo].abs().max().item() == 0 and mc.grad[..., hi:].abs().max().item() == 0


@pytest.mark.parametrize("case", ["2048", "small-blocks-ragged", "fp16-alpha", "dropout", "alibi", "window", "window-dropout"])
def test_blocked_causal_gemms_equal_the_dense_ones(case, monkeypatch):
    """With the causal kernel the score, context and gradient GEMMs are computed on and below the diagonal blocks
    only (nothing above is read, and the probabilities and their gradients are exact zeros there). Against the same
    module with dense GEMMs, and against fp32 textbook attention; the uninitialised parts of the score tensor are
    filled with NaN first to show that they are never used."""
    from megatron.model import attention_core
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    dtype = torch.float16 if case == "fp16-alpha" else torch.bfloat16
    sq, b, np_, hn = (2048, 1, 4, 64) if case == "2048" else (328, 2, 4, 64)
    if case != "2048":
        monkeypatch.setattr(attention_core, "causal_gemm_block", lambda s: 128)   # blocks of 128, 128 and 72 rows
    real_empty = torch.empty

    real_empty_like = torch.empty_like

    def poisoned_empty(*args, **kw):
        t = real_empty(*args, **kw)
        return t.fill_(float("nan")) if t.is_floating_point() else t

    def poisoned_empty_like(*args, **kw):   # the softmax outputs, of which the kernel writes only the blocks in use
        t = real_empty_like(*args, **kw)
        return t.fill_(float("nan")) if t.is_floating_point() else t

    kw = dict(attention_softmax_in_fp32=True)
    if case.endswith("dropout"):
        kw["attention_dropout"] = 0.1
    if case.startswith("window"):   # 100 keys: row blocks 2 and 3 start after key 0, and after key 128 for the last one
        kw["sliding_window_width"] = 100
    if case == "alibi":
        from megatron.model.positional_embeddings import AliBi
        kw["alibi_slopes"] = AliBi(np_, 1, 0).slopes
    fp16, bf16 = dtype == torch.float16, dtype == torch.bfloat16
    blocked = CoreAttention(hn, 1, fp16, bf16, T.upper_triang, mask_func, **kw).to(DEV)
    dense = CoreAttention(hn, 1, fp16, bf16, T.upper_triang, mask_func, causal_gemm_blocks=False, **kw).to(DEV)
    mask = fb.causal_mask(sq, DEV)
    if case.startswith("window"):
        pos = torch.arange(sq, device=DEV)
        mask = mask | (pos.view(1, 1, sq, 1) - pos.view(1, 1, 1, sq) > 100)
        assert attention_core._row_blocks(sq, 128, 100) == [(0, 128, 0), (128, 256, 0), (256, 328, 128)]
        assert attention_core._column_blocks(sq, 128, 100) == [(0, 128, 228), (128, 256, 328), (256, 328, 328)]
    q, k, v = qkv(dtype, sq, b, np_, hn, 51)
    q2, k2, v2 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
    assert blocked._causal_block(mask, b, np_, sq, sq, q) == (512 if case == "2048" else 128)
    assert dense._causal_block(mask, b, np_, sq, sq, q) == 0
    g = util.randn((sq, b, np_ * hn), dtype, seed=55).to(DEV)
    torch.manual_seed(7)
    monkeypatch.setattr(attention_core.torch, "empty", poisoned_empty)
    monkeypatch.setattr(attention_core.torch, "empty_like", poisoned_empty_like)
    out = blocked(q, k, v, mask, merged_heads=True)
    out.backward(g)
    monkeypatch.setattr(attention_core.torch, "empty", real_empty)
    monkeypatch.setattr(attention_core.torch, "empty_like", real_empty_like)
    torch.manual_seed(7)   # the same dropout seed for the second module
    out2 = dense(q2, k2, v2, mask, merged_heads=True)
    out2.backward(g)
    lim = 2.0 ** (-7 if dtype == torch.bfloat16 else -9)
    for got, want in ((out, out2), (q.grad, q2.grad), (k.grad, k2.grad), (v.grad, v2.grad)):
        assert torch.isfinite(got).all()
        assert rel_err(got, want) <= lim / 4
    if case in ("2048", "small-blocks-ragged", "fp16-alpha", "window"):
        q3, k3, v3 = (t.detach().clone().requires_grad_(True) for t in (q, k, v))
        ref = textbook(q3, k3, v3, mask).permute(2, 0, 1, 3).reshape(sq, b, np_ * hn)
        ref.backward(g.float())
        assert rel_err(out, ref) <= lim
        for got, want in ((q.grad, q3.grad), (k.grad, k3.grad), (v.grad, v3.grad)):
            assert rel_err(got, want) <= 2 * lim
    # the [b, np, sq, hn] result as well
    assert rel_err(blocked(q.detach(), k.detach(), v.detach(), mask).permute(2, 0, 1, 3).reshape(sq, b, np_ * hn)
                   if not case.endswith("dropout") else out, out) <= lim / 4
    # the dense GEMMs are kept where the causal kernel is not what runs
    general = CoreAttention(hn, 1, fp16, bf16, T.general, mask_func, **kw).to(DEV)
    assert general._causal_block(mask, b, np_, sq, sq, q) == 0
    assert blocked._causal_block(mask, b, np_, sq, sq + 8, q) == 0
