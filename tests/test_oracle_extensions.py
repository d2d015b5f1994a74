"""Pins the oracle's sliding-window and AliBi variants of the causal softmax and
the host-side AliBi mirror, without a GPU."""
import math

import pytest
import torch

import oracle
import util
from oracle import fallback_semantics as fb

DTYPES = [torch.bfloat16, torch.float16]
IDS = ["bf16", "fp16"]


def f64_softmax_rows(z):
    z = z.double()
    z = z - z.max(dim=-1, keepdim=True).values
    e = z.exp()
    return e / e.sum(dim=-1, keepdim=True)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("s,window", [(16, 0), (16, 3), (33, 8), (100, 31), (100, 99), (64, 200)])
def test_sliding_window_forward(dtype, s, window):
    a, scale = 2, 0.3
    x = util.randn((a, s, s), dtype, seed=s + window, std=2.0)
    y = oracle.causal_softmax_fwd(x, scale, window=window)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    # everything outside the band is +0 bit for bit
    assert int(util.raw_bits(y)[:, masked].abs().max()) == 0
    # float64 brute force over the band
    z = (x.double() * float(torch.tensor(scale, dtype=torch.float32))).masked_fill(masked, float("-inf"))
    util.assert_ulp_close(y, f64_softmax_rows(z).to(dtype), 1, "vs float64")
    # the reference's torch path with the sliding-window mask of get_attn_mask
    ref = fb.torch_softmax_fallback(x.view(1, a, s, s), masked.view(1, 1, s, s), scale).view(a, s, s)
    util.assert_ulp_close(y, ref, 1, "vs torch fallback")
    # the band of row q holds min(q, window) + 1 keys
    counts = (~masked).sum(-1)
    assert torch.equal(counts, torch.clamp(torch.arange(s), max=window) + 1)
    if window == 0:
        assert torch.equal(y.float(), torch.eye(s).expand(a, s, s))
    if window >= s - 1:
        assert torch.equal(util.raw_bits(y), util.raw_bits(oracle.causal_softmax_fwd(x, scale)))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_sliding_window_backward(dtype):
    a, s, window, scale = 2, 40, 9, 0.6
    x = util.randn((a, s, s), dtype, seed=1, std=2.0)
    y = oracle.causal_softmax_fwd(x, scale, window=window)
    dy = util.randn((a, s, s), dtype, seed=2)
    dx = oracle.softmax_bwd(dy, y, scale, causal=True, window=window)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    assert int(util.raw_bits(dx)[:, masked].abs().max()) == 0
    g = (dy.double() * y.double()).masked_fill(masked, 0.0)
    want = float(torch.tensor(scale, dtype=torch.float32)) * (g - y.double().masked_fill(masked, 0.0) * g.sum(-1, keepdim=True))
    util.assert_softmax_bwd_close(dx, want.to(dtype), dy.masked_fill(masked, 0), y, scale, "vs float64 JVP")
    # dy outside the band must not leak into the row sum: garbage there changes nothing
    dy2 = dy.clone()
    dy2[:, masked] = 1000.0
    dx2 = oracle.softmax_bwd(dy2, y, scale, causal=True, window=window)
    assert torch.equal(util.raw_bits(dx2), util.raw_bits(dx))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("heads", [4, 6])
def test_alibi_equals_eager_add_then_plain_softmax(dtype, heads):
    """softmax_alibi(x) == softmax(x + alibi_matrix) with the sum formed by torch in
    the storage dtype: pins the sign, the orientation (q - k), the head indexing
    (batch % heads) and the three roundings."""
    b, s, scale = 2, 300, 0.2  # distances above 256 are not exact in bf16
    slopes = torch.tensor(fb.alibi_slopes(heads), dtype=torch.float32)
    x = util.randn((b, heads, s, s), dtype, seed=heads, std=2.0)
    fused = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, alibi_slopes=slopes)
    eager = oracle.causal_softmax_fwd(fb.alibi_add(x, slopes).view(-1, s, s), scale)
    assert torch.equal(util.raw_bits(fused), util.raw_bits(eager))
    zero = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, alibi_slopes=torch.zeros(heads))
    assert torch.equal(util.raw_bits(zero), util.raw_bits(oracle.causal_softmax_fwd(x.view(-1, s, s), scale)))
    # the bias favours recent keys: with constant scores the probabilities increase towards the diagonal
    c = torch.zeros((1, heads, 64, 64), dtype=dtype)
    p = oracle.causal_softmax_fwd(c.view(-1, 64, 64), 1.0, alibi_slopes=slopes).float()
    assert (p[0, 63, :64].diff() >= 0).all() and p[0, 63, 63] > p[0, 63, 0]


def test_alibi_with_window_combined():
    heads, s, window = 4, 64, 10
    slopes = torch.tensor(fb.alibi_slopes(heads), dtype=torch.float32)
    x = util.randn((1, heads, s, s), torch.bfloat16, seed=3, std=2.0)
    fused = oracle.causal_softmax_fwd(x.view(-1, s, s), 0.5, window=window, alibi_slopes=slopes)
    eager = oracle.causal_softmax_fwd(fb.alibi_add(x, slopes).view(-1, s, s), 0.5, window=window)
    assert torch.equal(util.raw_bits(fused), util.raw_bits(eager))


def test_alibi_module_mirror():
    from megatron.model.positional_embeddings import AliBi

    # the reference's default mp_rank=1 with mp_size=1 selects an empty slice; callers pass the 0-based rank
    assert AliBi(8).slopes.numel() == 0
    a8 = AliBi(8, mp_size=1, mp_rank=0)
    assert torch.allclose(a8.slopes, torch.tensor([2.0 ** -(i + 1) for i in range(8)]))
    a12 = AliBi(12, 1, 0)
    assert a12.slopes.shape == (12,) and torch.allclose(a12.slopes, torch.tensor(fb.alibi_slopes(12)))
    assert torch.allclose(a12.slopes[:8], a8.slopes)
    # model-parallel slicing: rank r keeps heads [r*slice, (r+1)*slice)
    part = AliBi(8, mp_size=2, mp_rank=1)
    assert torch.equal(part.slopes, a8.slopes[4:])
    assert "slopes" in a8.state_dict()
    # forward adds -(q-k)*slope below the diagonal and nothing above
    x = torch.zeros(1, 8, 5, 5)
    y = a8(x)
    assert y[0, 0, 4, 0].item() == -4 * 0.5 and y[0, 0, 4, 4].item() == 0 and y[0, 0, 0, 4].item() == 0
    assert y[0, 3, 3, 1].item() == -2 * 2.0**-4
    # same arithmetic as the restatement, in bf16
    xb = util.randn((2, 8, 40, 40), torch.bfloat16, seed=1)
    assert torch.equal(util.raw_bits(AliBi(8, 1, 0)(xb)), util.raw_bits(fb.alibi_add(xb, a8.slopes)))
    # the cached matrix grows fourfold, is clipped for shorter inputs, and serves single-query decoding
    al = AliBi(4, 1, 0)
    al(torch.zeros(1, 4, 6, 6))
    assert al.cached_seq_len == 6
    al(torch.zeros(1, 4, 7, 7))
    assert al.cached_seq_len == 24
    assert al(torch.zeros(1, 4, 3, 3)).shape == (1, 4, 3, 3)
    d = al(torch.zeros(1, 4, 1, 9))
    assert d.shape == (1, 4, 1, 9) and d[0, 0, 0, 8].item() == 0 and d[0, 0, 0, 0].item() == -8 * al.slopes[0].item()
    with pytest.raises(AssertionError):
        al(torch.zeros(1, 4, 2, 9))


@pytest.mark.parametrize("dtype,fp16,bf16", [(torch.float16, True, False), (torch.bfloat16, False, True)])
def test_module_torch_path_with_window_and_alibi(dtype, fp16, bf16):
    """With fusion off the module applies the same semantics with torch ops (CPU here)."""
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T

    b, np_, s, window, scale = 2, 4, 48, 7, 0.25
    slopes = torch.tensor(fb.alibi_slopes(np_), dtype=torch.float32)
    x = util.randn((b, np_, s, s), dtype, seed=5, std=2.0)
    m = FusedScaleMaskSoftmax(fp16, bf16, T.none, fb.fill_masked_with_dtype_min, True, scale,
                              sliding_window_width=window, alibi_slopes=slopes)
    y = m(x.clone(), fb.causal_mask(s, sliding_window_width=window))
    want = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, window=window, alibi_slopes=slopes).view(b, np_, s, s)
    util.assert_ulp_close(y, want, 1, "torch path vs oracle")
    assert "alibi_slopes" not in m.state_dict()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_additive_bias_equals_eager_add_then_plain_softmax(dtype):
    """softmax_bias(x, bias) == softmax(x + bias) with the sum formed by torch in the
    storage dtype (`attention_scores += rpe`), the bias being shared by the batch and
    indexed by head; combined with AliBi the bias comes first."""
    b, heads, s, scale = 3, 4, 40, 0.3
    x = util.randn((b, heads, s, s), dtype, seed=1, std=2.0)
    bias = util.randn((1, heads, s, s), dtype, seed=2, std=1.5)
    fused = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, bias=bias[0])
    eager = oracle.causal_softmax_fwd((x + bias).view(-1, s, s), scale)
    assert torch.equal(util.raw_bits(fused), util.raw_bits(eager))
    assert not torch.equal(util.raw_bits(fused), util.raw_bits(oracle.causal_softmax_fwd(x.view(-1, s, s), scale)))
    slopes = torch.tensor(fb.alibi_slopes(heads), dtype=torch.float32)
    both = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, window=9, alibi_slopes=slopes, bias=bias[0])
    eager = oracle.causal_softmax_fwd(fb.alibi_add(x + bias, slopes).view(-1, s, s), scale, window=9)
    assert torch.equal(util.raw_bits(both), util.raw_bits(eager))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("window", [None, 6])
def test_key_lengths_forward(dtype, window):
    """Padding keys k >= len[b] masked by index: float64 brute force over the kept band,
    the torch fallback given the merged mask, rows the padding does not reach unchanged
    bit for bit, rows without any key uniform (1/s in every column, above the diagonal too, as the torch
    fallback's softmax over a row of equal fill values)."""
    batch, heads, s, scale = 4, 2, 40, 0.3
    lengths = torch.tensor([40, 13, 1, 0], dtype=torch.int32)
    x = util.randn((batch * heads, s, s), dtype, seed=5, std=2.0)
    y = oracle.causal_softmax_fwd(x, scale, window=window, key_lengths=lengths)
    plain = oracle.causal_softmax_fwd(x, scale, window=window)
    causal = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    keys = torch.arange(s)
    masked = (causal[None] | (keys[None, None, :] >= lengths.view(-1, 1, 1))).repeat_interleave(heads, dim=0)
    empty = masked.all(-1)
    assert empty[-heads:].all() and not empty[:heads].any()        # length 0 / full length
    assert int(util.raw_bits(y)[masked & ~empty[..., None]].abs().max()) == 0
    assert torch.equal(y[empty], torch.full_like(y[empty], 1.0 / s))
    z = (x.double() * float(torch.tensor(scale, dtype=torch.float32))).masked_fill(masked, float("-inf"))
    live = ~empty
    util.assert_ulp_close(y[live], f64_softmax_rows(z[live]).to(dtype), 1, "vs float64")
    ref = fb.torch_softmax_fallback(x.view(batch, heads, s, s), masked.view(batch, heads, s, s)[:, :1], scale)
    util.assert_ulp_close(y, ref.view(-1, s, s), 1, "vs torch fallback with the merged mask")   # empty rows included
    # a row whose causal band ends before the padding starts is the plain row
    q = torch.arange(s)
    untouched = (q[None, :] < lengths.view(-1, 1)).repeat_interleave(heads, dim=0)
    assert torch.equal(util.raw_bits(y)[untouched], util.raw_bits(plain)[untouched])
    assert not torch.equal(util.raw_bits(y)[live & ~untouched], util.raw_bits(plain)[live & ~untouched])
    # lengths beyond the row change nothing; negative ones count as zero
    assert torch.equal(util.raw_bits(oracle.causal_softmax_fwd(x, scale, window=window,
                                                               key_lengths=torch.tensor([99, 40, 41, 1000]))),
                       util.raw_bits(plain))
    none = oracle.causal_softmax_fwd(x, scale, key_lengths=torch.tensor([-1, -5, 0, -2]))
    assert torch.equal(none, torch.full_like(none, 1.0 / s))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_key_lengths_backward(dtype):
    """dx = scale * y * (dy - sum_kept(dy * y)) on the kept band, +0 elsewhere: float64
    evaluation of the Jacobian-vector product from the rounded y, and autograd through
    the float64 softmax with the merged mask."""
    batch, heads, s, scale = 3, 2, 24, 0.7
    lengths = torch.tensor([24, 9, 0], dtype=torch.int32)
    x = util.randn((batch * heads, s, s), dtype, seed=6, std=1.5)
    dy = util.randn((batch * heads, s, s), dtype, seed=7)
    y = oracle.causal_softmax_fwd(x, scale, key_lengths=lengths)
    dx = oracle.softmax_bwd(dy, y, scale, causal=True, key_lengths=lengths)
    keys = torch.arange(s)
    masked = (fb.causal_mask(s)[0, 0][None] | (keys[None, None, :] >= lengths.view(-1, 1, 1))).repeat_interleave(heads, dim=0)
    assert int(util.raw_bits(dx)[masked].abs().max()) == 0
    yd, gd = y.double().masked_fill(masked, 0), dy.double().masked_fill(masked, 0)
    f32scale = float(torch.tensor(scale, dtype=torch.float32))
    want = f32scale * yd * (gd - (gd * yd).sum(-1, keepdim=True))
    util.assert_softmax_bwd_close(dx, want.to(dtype), dy.masked_fill(masked, 0), y, scale, "vs float64 formula")
    # autograd of the float64 softmax (exact y instead of the rounded one: looser)
    live = ~masked.all(-1)
    xd = x.double().requires_grad_(True)
    p = torch.softmax((xd * f32scale).masked_fill(masked, float("-inf"))[live], -1)
    p.backward(dy.double()[live])
    err = (dx.double()[live] - xd.grad[live]).abs().max().item()
    assert err <= 3 * 2.0 ** (-8 if dtype == torch.bfloat16 else -11) * xd.grad.abs().max().item()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("window", [None, 5])
def test_softmax_with_attention_dropout_is_the_composition(dtype, window):
    """softmax + dropout in one function == the softmax oracle followed by torch's definition of
    dropout (keep ? v / (1 - p) : 0 on the stored probabilities) with the oracle's mask; the backward
    == the dropout backward followed by the softmax backward, and matches float64 autograd."""
    a, s, scale, p, seed = 3, 24, 0.4, 0.3, 77
    x = util.randn((a, s, s), dtype, seed=1, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=2)
    dropped, y = oracle.causal_softmax_dropout_fwd(x, scale, p, seed, window=window)
    plain = oracle.causal_softmax_fwd(x, scale, window=window)
    assert torch.equal(util.raw_bits(y), util.raw_bits(plain))
    keep = oracle.dropout_mask(x.numel(), p, seed).view_as(x)
    ds = torch.tensor(1.0 / (1.0 - p), dtype=torch.float64).float()
    want = torch.where(keep, plain.float() * ds, torch.zeros(())).to(dtype)
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(want))
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(plain, None, None, p, seed)))
    dx = oracle.causal_softmax_dropout_bwd(dy, y, scale, p, seed, window=window)
    g = oracle.bias_dropout_add(dy, None, None, p, seed)       # the dropout backward, stored in the dtype
    assert torch.equal(util.raw_bits(dx), util.raw_bits(oracle.softmax_bwd(g, y, scale, True, window=window)))
    # float64 autograd through softmax and the same mask (exact y instead of the rounded one: looser)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    xd = x.double().requires_grad_(True)
    f32scale = float(torch.tensor(scale, dtype=torch.float32))
    probs = torch.softmax((xd * f32scale).masked_fill(masked, float("-inf")), -1)
    (probs * keep / (1 - p)).backward(dy.double())
    err = (dx.double() - xd.grad).abs().max().item()
    assert err <= 4 * 2.0 ** (-8 if dtype == torch.bfloat16 else -11) * xd.grad.abs().max().item()
    # p = 0 is the plain pair
    d0, y0 = oracle.causal_softmax_dropout_fwd(x, scale, 0.0, seed, window=window)
    assert torch.equal(util.raw_bits(d0), util.raw_bits(plain)) and torch.equal(util.raw_bits(y0), util.raw_bits(plain))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_masked_softmax_with_attention_dropout_is_the_composition(dtype):
    """The padding-mask softmax followed by dropout: the probabilities are those of masked_softmax_fwd, the
    dropped tensor equals the C oracle's dropout of them (one shared mask definition over the flat index), the
    backward is the dropout backward followed by the unmasked softmax backward and matches float64 autograd
    on the rows that are not fully masked."""
    b, np_, sq, sk, scale, p, seed = 3, 2, 5, 24, 0.4, 0.3, 91
    x = util.randn((b, np_, sq, sk), dtype, seed=1, std=2.0)
    dy = util.randn((b, np_, sq, sk), dtype, seed=2)
    mask = util.padding_mask(b, sq, sk, seed=3, full_batch=1, lo=4)
    dropped, y = oracle.masked_softmax_dropout_fwd(x, mask, scale, p, seed)
    plain = oracle.masked_softmax_fwd(x, mask, scale)
    assert torch.equal(util.raw_bits(y), util.raw_bits(plain))
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(plain, None, None, p, seed)))
    keep = oracle.dropout_mask(x.numel(), p, seed).view_as(x)
    assert dropped[~keep].abs().max().item() == 0
    dx = oracle.masked_softmax_dropout_bwd(dy, y, scale, p, seed)
    g = oracle.bias_dropout_add(dy, None, None, p, seed)
    assert torch.equal(util.raw_bits(dx), util.raw_bits(oracle.softmax_bwd(g, y, scale, False)))
    xd = x.double().requires_grad_(True)
    f32scale = float(torch.tensor(scale, dtype=torch.float32))
    full = mask.expand(b, np_, sq, sk)
    probs = torch.softmax((xd * f32scale).masked_fill(full, -10000.0), -1)
    (probs * keep / (1 - p)).backward(dy.double())
    live = ~mask.all(dim=-1, keepdim=True).expand_as(x)       # fully masked rows: the kernel backward has no mask
    err = ((dx.double() - xd.grad).abs() * live).max().item()
    assert err <= 4 * 2.0 ** (-8 if dtype == torch.bfloat16 else -11) * xd.grad.abs().max().item()
    d0, y0 = oracle.masked_softmax_dropout_fwd(x, mask, scale, 0.0, seed)
    assert torch.equal(util.raw_bits(d0), util.raw_bits(plain)) and torch.equal(util.raw_bits(y0), util.raw_bits(plain))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_padding_mask_softmax_with_extras_is_the_composition(dtype):
    """The padding-mask softmax with a bias tensor, AliBi slopes and key lengths is the plain one on operands
    prepared by the caller's eager statements (transformer.py:580-588). Two independent statements must meet:
    given the causal mask, it equals the causal kernel semantics (C) with the same extras on every row (a row
    without keys is 1/sk in both): exact zeros in the same places, and probabilities within 1 ulp (the two sum
    a row's exponentials over different lengths, hence in a different order)."""
    b, heads, s, scale = 3, 4, 72, 0.3
    slopes = torch.tensor(fb.alibi_slopes(heads), dtype=torch.float32)
    x = util.randn((b, heads, s, s), dtype, seed=11, std=2.0)
    bias = util.randn((heads, s, s), dtype, seed=12, std=1.5)
    lengths = torch.tensor([s, 29, 0], dtype=torch.int32)
    mask = fb.causal_mask(s)
    for use_slopes, use_bias, use_len in [(1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 1, 1)]:
        kw = dict(alibi_slopes=slopes if use_slopes else None, bias=bias if use_bias else None,
                  key_lengths=lengths if use_len else None)
        general = oracle.masked_softmax_fwd(x, mask, scale, **kw)
        causal = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, **kw).view_as(x)
        assert torch.equal(util.raw_bits(general) == 0, util.raw_bits(causal) == 0)
        util.assert_ulp_close(general, causal, 1, str((use_slopes, use_bias, use_len)))
        if use_len:
            # the sequence without any key: every row uniform, exactly fl(1/sk)
            assert torch.equal(general[2], torch.full_like(general[2], 1.0 / s))
    # the prepared operands themselves: in-place add, AliBi.forward, merged padding
    xs, m = oracle.prepared_masked_inputs(x, mask, slopes, bias, lengths)
    assert torch.equal(util.raw_bits(xs), util.raw_bits(fb.alibi_add(x + bias, slopes)))
    assert bool(m[1, 0, :, 29:].all()) and not bool(m[1, 0, 40, :29].any()) and bool(m[2].all())
    assert torch.equal(m[0], mask[0])
    # a [b, 1, sq, sk] mask and a uint8 mask work the same
    per_batch = mask.expand(b, 1, s, s).contiguous()
    a = oracle.masked_softmax_fwd(x, per_batch.to(torch.uint8), scale, slopes, bias, lengths)
    assert torch.equal(util.raw_bits(a), util.raw_bits(oracle.masked_softmax_fwd(x, mask, scale, slopes, bias, lengths)))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rectangular_scores_with_bias_and_key_lengths(dtype):
    """sq != sk (new positions after cached keys): bias and key lengths against float64 brute force."""
    b, heads, sq, sk, scale = 2, 3, 5, 40, 0.25
    x = util.randn((b, heads, sq, sk), dtype, seed=21, std=2.0)
    bias = util.randn((heads, sq, sk), dtype, seed=22)
    lengths = torch.tensor([33, 40], dtype=torch.int32)
    mask = util.padding_mask(b, sq, sk, seed=23, lo=20)
    got = oracle.masked_softmax_fwd(x, mask, scale, bias=bias, key_lengths=lengths)
    z = (x + bias).double() * float(torch.tensor(scale, dtype=torch.float32))
    full = mask.expand(b, heads, sq, sk) | (torch.arange(sk).view(1, 1, 1, sk) >= lengths.view(b, 1, 1, 1))
    want = f64_softmax_rows(z.masked_fill(full, -10000.0))
    util.assert_ulp_close(got, want.to(dtype), 1, "rectangular")
    assert int(util.raw_bits(got)[full & ~full.all(-1, keepdim=True)].abs().max()) == 0


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_causal_softmax_dropout_with_extras_is_the_composition(dtype):
    """Dropout after the causal softmax with extras: same probabilities as without dropout, dropped = the C
    oracle's dropout of them; with trivial extras the composed route equals the single C function."""
    b, heads, s, scale, p, seed = 2, 2, 40, 0.3, 0.25, 77
    x = util.randn((b * heads, s, s), dtype, seed=31, std=2.0)
    dy = util.randn((b * heads, s, s), dtype, seed=32)
    slopes = torch.tensor(fb.alibi_slopes(heads), dtype=torch.float32)
    bias = util.randn((heads, s, s), dtype, seed=33)
    lengths = torch.tensor([s, 17], dtype=torch.int32)
    dropped, y = oracle.causal_softmax_dropout_fwd(x, scale, p, seed, window=9, alibi_slopes=slopes, bias=bias,
                                                   key_lengths=lengths)
    plain = oracle.causal_softmax_fwd(x, scale, window=9, alibi_slopes=slopes, bias=bias, key_lengths=lengths)
    assert torch.equal(util.raw_bits(y), util.raw_bits(plain))
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(plain, None, None, p, seed)))
    # zero bias: the composed route against the C function that does softmax and dropout at once
    d1, y1 = oracle.causal_softmax_dropout_fwd(x, scale, p, seed, window=9, bias=torch.zeros_like(bias))
    d2, y2 = oracle.causal_softmax_dropout_fwd(x, scale, p, seed, window=9)
    assert torch.equal(util.raw_bits(d1), util.raw_bits(d2)) and torch.equal(util.raw_bits(y1), util.raw_bits(y2))
    # backward: all lengths full = the C function; shorter lengths zero the padding columns
    full = torch.tensor([s, s], dtype=torch.int32)
    g1 = oracle.causal_softmax_dropout_bwd(dy, y2, scale, p, seed, window=9, key_lengths=full)
    g2 = oracle.causal_softmax_dropout_bwd(dy, y2, scale, p, seed, window=9)
    assert torch.equal(util.raw_bits(g1), util.raw_bits(g2))
    g3 = oracle.causal_softmax_dropout_bwd(dy, y, scale, p, seed, window=9, key_lengths=lengths)
    assert int(util.raw_bits(g3)[heads:, :, 17:].abs().max()) == 0
