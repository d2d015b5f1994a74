"""GPU parity of the sliding-window / AliBi variants of the causal softmax, through
the C ABI and through FusedScaleMaskSoftmax, against the CPU oracle.
Tolerances as for the plain kernels: 2 ulp forward, masked positions bit-exact +0,
backward 2 ulp plus the fp32 row-sum noise."""
import math

import pytest
import torch

import oracle
import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.bfloat16, torch.float16]


def abi_ex_fwd(hp, x, scale, window, slopes, bias=None, key_lengths=None):
    y = torch.empty_like(x)
    heads = slopes.numel() if slopes is not None else bias.size(0) if bias is not None else 1
    if key_lengths is not None:
        assert key_lengths.dtype == torch.int32
        heads = x.size(0) // key_lengths.numel()
    rc = hp.lib().nhp_causal_softmax_ex_fwd(
        y.data_ptr(), x.data_ptr(), scale, x.size(0), x.size(1), -1 if window is None else window,
        None if slopes is None else slopes.data_ptr(), None if bias is None else bias.data_ptr(),
        None if key_lengths is None else key_lengths.data_ptr(), heads, hp.dtype_code(x, "t"), None)
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return y


def abi_ex_bwd(hp, dy, y, scale, window, key_lengths=None):
    dx = torch.empty_like(dy)
    heads = 1 if key_lengths is None else dy.size(0) // key_lengths.numel()
    rc = hp.lib().nhp_causal_softmax_ex_bwd(dx.data_ptr(), dy.data_ptr(), y.data_ptr(), scale, dy.size(0), dy.size(1),
                                            -1 if window is None else window,
                                            None if key_lengths is None else key_lengths.data_ptr(), heads,
                                            hp.dtype_code(dy, "t"), None)
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return dx


# (attn_batches, seq_len, window, heads or None)
CASES = [
    (4, 64, 0, None), (4, 64, 5, 2), (3, 200, 63, None), (2, 512, 100, 2), (2, 1024, 511, None),
    (2, 1024, 512, 2), (2, 2048, 7, None), (6, 2048, 700, 6), (2, 2048, None, 2), (1, 4096, 1000, None),
    (2, 4096, 3000, 2), (1, 8192, 2047, 1), (2, 1001, 50, 2), (2, 33, 40, None), (4, 2056, 1024, 4),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"a{c[0]}_s{c[1]}_w{c[2]}_h{c[3]}")
def test_window_alibi_forward_backward_vs_oracle(hotpath, case, dtype):
    a, s, window, heads = case
    print(f"ex case {case} {dtype}", flush=True)
    scale = 1 / math.sqrt(128)
    slopes = None if heads is None else torch.tensor(fb.alibi_slopes(max(heads, 2))[:heads], dtype=torch.float32)
    x = util.randn((a, s, s), dtype, seed=s + (window or 0), std=2.0)
    dy = util.randn((a, s, s), dtype, seed=s + 1)
    want_y = oracle.causal_softmax_fwd(x, scale, window=window, alibi_slopes=slopes)
    got_y = abi_ex_fwd(hotpath, x.to(DEV), scale, window, None if slopes is None else slopes.to(DEV)).cpu()
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    assert int(util.raw_bits(got_y)[:, masked].abs().max() if masked.any() else 0) == 0
    util.assert_ulp_close(got_y, want_y, 2, "fwd")
    want_dx = oracle.softmax_bwd(dy, want_y, scale, causal=True, window=window)
    got_dx = abi_ex_bwd(hotpath, dy.to(DEV), want_y.to(DEV), scale, window).cpu()
    assert int(util.raw_bits(got_dx)[:, masked].abs().max() if masked.any() else 0) == 0
    util.assert_softmax_bwd_close(got_dx, want_dx, dy.masked_fill(masked, 0), want_y, scale, "bwd")


def test_window_never_reads_outside_the_band(hotpath):
    """NaNs planted outside the band (and above the diagonal) must not reach the output."""
    a, s, window = 2, 2048, 300
    x = util.randn((a, s, s), torch.bfloat16, seed=1, std=2.0)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    # chunk granularity: a 16-byte chunk that straddles the band edge is loaded, so poison whole chunks only
    col = torch.arange(s)
    q = torch.arange(s)[:, None]
    poison = ((col[None, :] // 8 * 8 + 8) <= (q - window)) | ((col[None, :] // 8 * 8) > q)
    xp = x.clone()
    xp[:, poison] = float("nan")
    y = abi_ex_fwd(hotpath, xp.to(DEV), 0.1, window, None).cpu()
    assert not torch.isnan(y.float()).any()
    util.assert_ulp_close(y, oracle.causal_softmax_fwd(x, 0.1, window=window), 2, "poisoned")


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_module_with_window_and_alibi(dtype):
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T
    from megatron.model.positional_embeddings import AliBi

    b, np_, s, window, scale = 2, 8, 1024, 256, 0.125
    alibi = AliBi(np_, mp_size=1, mp_rank=0)
    x = util.randn((b, np_, s, s), dtype, seed=9, std=2.0)
    dy = util.randn((b, np_, s, s), dtype, seed=10)
    mask = fb.causal_mask(s, DEV, sliding_window_width=window)
    fused = FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, T.upper_triang,
                                  fb.fill_masked_with_dtype_min, True, scale, sliding_window_width=window,
                                  alibi_slopes=alibi.slopes).to(DEV)
    xd = x.to(DEV).requires_grad_(True)
    y = fused(xd, mask)
    want = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, window=window, alibi_slopes=alibi.slopes).view(b, np_, s, s)
    util.assert_ulp_close(y.detach().cpu(), want, 2, "module fwd")
    y.backward(dy.to(DEV))
    yc = y.detach().cpu()
    want_dx = oracle.softmax_bwd(dy.view(-1, s, s), yc.view(-1, s, s), scale, True, window=window).view(b, np_, s, s)
    masked = mask.cpu()[0, 0]
    util.assert_softmax_bwd_close(xd.grad.cpu(), want_dx, dy.masked_fill(masked, 0), yc, scale, "module bwd")
    # the unfused route the reference would take: eager AliBi add, then the torch softmax with the window mask
    plain = FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, T.none,
                                  fb.fill_masked_with_dtype_min, True, scale)
    ref = plain(alibi.to(DEV)(x.to(DEV)), mask)
    util.assert_ulp_close(y.detach().cpu(), ref.cpu(), 2, "fused vs eager AliBi + torch softmax")


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("s,window,with_alibi", [(64, None, False), (1024, None, True), (2048, 300, False), (1001, None, False)])
def test_additive_bias_forward_vs_oracle(hotpath, dtype, s, window, with_alibi):
    import scaled_upper_triang_masked_softmax_cuda as ext

    b, heads, scale = 2, 4, 0.125
    x = util.randn((b * heads, s, s), dtype, seed=s, std=2.0)
    bias = util.randn((heads, s, s), dtype, seed=s + 1, std=1.5)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    slopes = torch.tensor(fb.alibi_slopes(heads), dtype=torch.float32) if with_alibi else None
    clean = oracle.causal_softmax_fwd(x, scale, window=window, alibi_slopes=slopes, bias=bias)
    # whatever lies outside the band, in the scores or in the bias, must not reach the result
    x[:, masked] = float("nan")
    bias[:, masked] = float("inf")
    want = oracle.causal_softmax_fwd(x, scale, window=window, alibi_slopes=slopes, bias=bias)
    assert torch.equal(util.raw_bits(clean), util.raw_bits(want))
    got = ext.forward(x.to(DEV), scale, window, None if slopes is None else slopes.to(DEV), bias.to(DEV)).cpu()
    assert int(util.raw_bits(got)[:, masked].abs().max()) == 0
    util.assert_ulp_close(got, want, 2, "bias fwd")
    via_abi = abi_ex_fwd(hotpath, x.to(DEV), scale, window, None if slopes is None else slopes.to(DEV), bias.to(DEV)).cpu()
    assert torch.equal(util.raw_bits(via_abi), util.raw_bits(got))


@pytest.mark.parametrize("b,heads,s", [(3, 2, 512), (5, 1, 1024), (2, 3, 2048), (3, 2, 4096), (3, 2, 200)])
def test_bias_shared_by_the_batch_workgroup_order(hotpath, b, heads, s):
    """With a bias tensor and more than one batch entry the forward kernels take the matrices in the order
    (head, batch entry), so that the matrices sharing a head's bias follow each other and find it in cache;
    batch sizes that are not powers of two, one head, rows of several waves, and a row count that does not
    fill its last workgroup (plain order). Every matrix against the oracle, causal and padding-mask kernel."""
    import scaled_masked_softmax_cuda as masked_ext
    import scaled_upper_triang_masked_softmax_cuda as ext

    dtype, scale = torch.bfloat16, 0.11
    print(f"shared bias b={b} heads={heads} s={s}", flush=True)
    x = util.randn((b * heads, s, s), dtype, seed=s + b, std=2.0)
    bias = util.randn((heads, s, s), dtype, seed=s + 1, std=1.5)
    want = oracle.causal_softmax_fwd(x, scale, bias=bias)
    got = ext.forward(x.to(DEV), scale, None, None, bias.to(DEV)).cpu()
    util.assert_ulp_close(got, want, 2, "causal, shared bias")
    sq = s // 8
    xm = util.randn((b, heads, sq, s), dtype, seed=s + b + 1, std=2.0)
    bm = util.randn((heads, sq, s), dtype, seed=s + 2, std=1.5)
    mask = util.padding_mask(b, sq, s, seed=s, lo=s // 2)
    want = oracle.masked_softmax_fwd(xm, mask, scale, None, bm, None)
    got = masked_ext.forward(xm.to(DEV), mask.to(DEV), scale, None, bm.to(DEV)).cpu()
    util.assert_ulp_close(got, want, 2, "padding mask, shared bias")


def test_module_with_relative_position_bias_and_its_gradient():
    """FusedScaleMaskSoftmax(input, mask, bias): probabilities and the gradients of the
    scores and of the (batch-shared, learned) bias against autograd through the unfused path."""
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T

    dtype = torch.bfloat16
    b, np_, s, scale = 3, 4, 512, 0.125
    x = util.randn((b, np_, s, s), dtype, seed=1, std=2.0)
    rpe = util.randn((1, np_, s, s), dtype, seed=2, std=1.0)
    dy = util.randn((b, np_, s, s), dtype, seed=3)
    mask = fb.causal_mask(s, DEV)
    out = {}
    for name, fusion in (("fused", T.upper_triang), ("plain", T.none)):
        m = FusedScaleMaskSoftmax(False, True, fusion, fb.fill_masked_with_dtype_min, True, scale)
        xd = x.to(DEV).requires_grad_(True)
        bd = rpe.to(DEV).requires_grad_(True)
        y = m(xd, mask, bd)
        y.backward(dy.to(DEV).clone())
        out[name] = (y.detach().cpu(), xd.grad.float().cpu(), bd.grad.float().cpu())
    want = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, bias=rpe[0]).view(b, np_, s, s)
    util.assert_ulp_close(out["fused"][0], want, 2, "fwd vs oracle")
    util.assert_ulp_close(out["fused"][0], out["plain"][0], 2, "fwd vs unfused")
    eps = 2.0**-8
    for i, what in ((1, "dx"), (2, "dbias")):
        f, p = out["fused"][i], out["plain"][i]
        assert (f - p).norm().item() <= 4 * eps * p.norm().item(), what
    assert out["fused"][2].shape == (1, np_, s, s)


def padded_mask(s, lengths, window=None):
    """[batch, s, s] bool, True = masked: above the diagonal, outside the window, or a padding key."""
    causal = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    keys = torch.arange(s)
    return causal[None] | (keys[None, None, :] >= lengths.view(-1, 1, 1))


# (batch, heads, seq_len, window, lengths)
LENGTH_CASES = [
    (4, 2, 64, None, [0, 1, 64, 37]),
    (3, 2, 512, None, [512, 100, 511]),
    (2, 3, 2048, None, [1500, 7]),
    (2, 2, 2048, 300, [2048, 1111]),       # rows 1411.. keep no key: the window starts in the padding
    (2, 2, 512, 8, [100, 101]),
    (2, 1, 4096, None, [4000, 513]),
    (2, 2, 1001, None, [1001, 333]),       # row length not a multiple of 8: scalar kernels
    (2, 2, 200, 17, [5000, -3]),           # out-of-range lengths clamp to [0, s]
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", LENGTH_CASES, ids=lambda c: f"b{c[0]}_h{c[1]}_s{c[2]}_w{c[3]}")
def test_key_lengths_forward_backward_vs_oracle(hotpath, case, dtype):
    batch, heads, s, window, lengths = case
    print(f"key-length case {case} {dtype}", flush=True)
    scale = 1 / math.sqrt(128)
    lengths = torch.tensor(lengths, dtype=torch.int32)
    x = util.randn((batch * heads, s, s), dtype, seed=s, std=2.0)
    dy = util.randn((batch * heads, s, s), dtype, seed=s + 1)
    masked = padded_mask(s, lengths, window).repeat_interleave(heads, dim=0)
    want_y = oracle.causal_softmax_fwd(x, scale, window=window, key_lengths=lengths)
    # the padding keys are never read: poison them (whole 16-byte chunks beyond the length)
    chunk_start = torch.arange(s) // 8 * 8
    beyond = (chunk_start[None, None, :] >= lengths.clamp(0, s).view(-1, 1, 1)).repeat_interleave(heads, dim=0)
    xp = x.clone()
    xp[beyond.expand_as(xp)] = float("nan")
    got_y = abi_ex_fwd(hotpath, xp.to(DEV), scale, window, None, None, lengths.to(DEV)).cpu()
    empty = masked.all(-1)                      # rows without any key: uniform, as on the torch branch
    assert int(util.raw_bits(got_y)[masked & ~empty[..., None]].abs().max()) == 0
    if empty.any():
        assert torch.equal(got_y[empty], torch.full_like(got_y[empty], 1.0 / s))
    util.assert_ulp_close(got_y, want_y, 2, "fwd")
    want_dx = oracle.softmax_bwd(dy, want_y, scale, causal=True, window=window, key_lengths=lengths)
    got_dx = abi_ex_bwd(hotpath, dy.to(DEV), want_y.to(DEV), scale, window, lengths.to(DEV)).cpu()
    assert int(util.raw_bits(got_dx)[masked].abs().max()) == 0
    util.assert_softmax_bwd_close(got_dx, want_dx, dy.masked_fill(masked, 0), want_y, scale, "bwd")


@pytest.mark.parametrize("fusion", ["upper_triang", "general"])
def test_module_with_key_lengths_all_branches_agree(fusion):
    """forward(input, mask, key_lengths=...) on a fused branch against the torch branch given
    the same arguments, probabilities and score gradients."""
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T

    dtype, b, np_, s, scale = torch.bfloat16, 4, 4, 512, 0.125
    lengths = torch.tensor([512, 300, 17, 450], device=DEV)
    x = util.randn((b, np_, s, s), dtype, seed=1, std=2.0)
    dy = util.randn((b, np_, s, s), dtype, seed=2)
    mask = fb.causal_mask(s, DEV)
    out = {}
    for name, kind in (("fused", T[fusion]), ("plain", T.none)):
        m = FusedScaleMaskSoftmax(False, True, kind, fb.fill_masked_with_dtype_min, True, scale)
        xd = x.to(DEV).requires_grad_(True)
        y = m(xd, mask, key_lengths=lengths)
        y.backward(dy.to(DEV).clone())
        out[name] = (y.detach().cpu(), xd.grad.float().cpu())
    masked = padded_mask(s, lengths.cpu())[:, None].expand(b, np_, s, s)
    util.assert_ulp_close(out["fused"][0], out["plain"][0], 2, "fwd fused vs torch branch")
    assert int(util.raw_bits(out["fused"][0])[masked].abs().max()) == 0
    f, p = out["fused"][1], out["plain"][1]
    assert (f - p).norm().item() <= 4 * 2.0**-8 * p.norm().item()
    if fusion == "upper_triang":
        want = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, key_lengths=lengths.cpu()).view(b, np_, s, s)
        util.assert_ulp_close(out["fused"][0], want, 2, "fwd vs oracle")


# (attn_batches, seq_len, window)
DROPOUT_CASES = [(4, 64, None), (3, 200, 63), (2, 512, None), (2, 1024, 100), (6, 2048, None), (1, 4096, 1000),
                 (1, 8192, None), (2, 1001, None), (2, 33, 7)]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", DROPOUT_CASES, ids=lambda c: f"a{c[0]}_s{c[1]}_w{c[2]}")
def test_softmax_with_attention_dropout_vs_oracle(hotpath, case, dtype):
    """Probabilities within 2 ulp of the oracle; the dropped tensor is exactly dropout (oracle mask) of the
    probabilities the GPU stored; the backward against the oracle given the same y."""
    import scaled_upper_triang_masked_softmax_cuda as ext

    a, s, window = case
    print(f"softmax+dropout case {case} {dtype}", flush=True)
    scale, p, seed = 1 / math.sqrt(128), 0.1, 1234 + s
    x = util.randn((a, s, s), dtype, seed=s, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=s + 1)
    want_y = oracle.causal_softmax_fwd(x, scale, window=window)
    dropped, y = [t.cpu() for t in ext.forward_dropout(x.to(DEV), scale, p, seed, window)]
    util.assert_ulp_close(y, want_y, 2, "y")
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    assert int(util.raw_bits(y)[:, masked].abs().max()) == 0 and int(util.raw_bits(dropped)[:, masked].abs().max()) == 0
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(y, None, None, p, seed)))
    want_dx = oracle.causal_softmax_dropout_bwd(dy, want_y, scale, p, seed, window=window)
    got_dx = ext.backward_dropout(dy.to(DEV).clone(), want_y.to(DEV), scale, p, seed, window).cpu()
    assert int(util.raw_bits(got_dx)[:, masked].abs().max()) == 0
    g = oracle.bias_dropout_add(dy, None, None, p, seed)
    util.assert_softmax_bwd_close(got_dx, want_dx, g.masked_fill(masked, 0), want_y, scale, "bwd")


def test_module_with_attention_dropout():
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T

    dtype, b, np_, s, scale, p = torch.bfloat16, 2, 4, 512, 0.125, 0.2
    x = util.randn((b, np_, s, s), dtype, seed=1, std=2.0)
    dy = util.randn((b, np_, s, s), dtype, seed=2)
    mask = fb.causal_mask(s, DEV)
    m = FusedScaleMaskSoftmax(False, True, T.upper_triang, fb.fill_masked_with_dtype_min, True, scale, attention_dropout=p)
    from megatron.model import dropout_rng

    torch.manual_seed(3)
    seed = dropout_rng.next_seed()  # what the module will draw
    torch.manual_seed(3)
    xd = x.to(DEV).requires_grad_(True)
    out = m(xd, mask)
    out.backward(dy.to(DEV).clone())
    want_d, want_y = oracle.causal_softmax_dropout_fwd(x.view(-1, s, s), scale, p, seed)
    keep = oracle.dropout_mask(x.numel(), p, seed).view(-1, s, s)
    got = out.detach().cpu().view(-1, s, s)
    assert int(util.raw_bits(got)[~keep].abs().max()) == 0
    assert (got.float() - want_d.float()).abs().max().item() <= 2.0**-7 * want_d.float().abs().max().item()
    want_dx = oracle.causal_softmax_dropout_bwd(dy.view(-1, s, s), want_y, scale, p, seed)
    gx = xd.grad.cpu().view(-1, s, s).float()
    assert (gx - want_dx.float()).norm().item() <= 2.0**-6 * want_dx.float().norm().item()
    # evaluation mode: no dropout, the plain kernel
    m.eval()
    util.assert_ulp_close(m(x.to(DEV), mask).cpu().view(-1, s, s), oracle.causal_softmax_fwd(x.view(-1, s, s), scale), 2, "eval")
    # the general-mask branch has its own fused kernel: same mask definition over the [b, np, sq, sk] tensor
    g = FusedScaleMaskSoftmax(False, True, T.general, fb.fill_masked_with_dtype_min, True, scale, attention_dropout=p)
    torch.manual_seed(3)
    xg = x.to(DEV).requires_grad_(True)
    yg = g(xg, mask)
    yg.backward(dy.to(DEV).clone())
    want_gd, want_gy = oracle.masked_softmax_dropout_fwd(x, mask.cpu(), scale, p, seed)
    keep4 = keep.view(b, np_, s, s)
    assert int(util.raw_bits(yg.detach().cpu())[~keep4].abs().max()) == 0
    assert (yg.detach().cpu().float() - want_gd.float()).abs().max().item() <= 2.0**-7 * want_gd.float().abs().max().item()
    want_gdx = oracle.masked_softmax_dropout_bwd(dy, want_gy, scale, p, seed)
    assert (xg.grad.cpu().float() - want_gdx.float()).norm().item() <= 2.0**-6 * want_gdx.float().norm().item()
    # with a bias it is still one kernel, and the same rate
    yb = g(x.to(DEV), mask, bias=torch.zeros((1, np_, s, s), dtype=dtype, device=DEV))
    zero_rate = ((yb == 0) & ~mask).float().sum().item() / (~mask).expand_as(yb).float().sum().item()
    assert abs(zero_rate - p) < 0.02


# (b, np, sq, sk): every forward geometry of the padding-mask kernel incl. the scalar fallback, both mask layouts
MASKED_DROPOUT_CASES = [(2, 3, 8, 64), (3, 2, 5, 200), (2, 2, 12, 512), (4, 2, 4, 1024), (2, 4, 16, 2048), (1, 2, 4, 4096),
                        (1, 2, 2, 8192), (2, 2, 6, 1001), (2, 1, 3, 24)]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("pad_batches", ["one", "each"])
@pytest.mark.parametrize("case", MASKED_DROPOUT_CASES, ids=lambda c: "x".join(map(str, c)))
def test_masked_softmax_with_attention_dropout_vs_oracle(hotpath, case, pad_batches, dtype):
    """As the causal test above, for the padding-mask kernel: probabilities within 2 ulp, the dropped tensor exactly
    the oracle's dropout of the stored probabilities, the backward against the oracle given the same y."""
    import scaled_masked_softmax_cuda as ext

    b, np_, sq, sk = case
    print(f"masked softmax+dropout case {case} {pad_batches} {dtype}", flush=True)
    scale, p, seed = 1 / math.sqrt(128), 0.15, 4321 + sk
    x = util.randn((b, np_, sq, sk), dtype, seed=sk, std=2.0)
    dy = util.randn((b, np_, sq, sk), dtype, seed=sk + 1)
    mask = util.padding_mask(b, sq, sk, seed=sk, full_batch=b - 1, lo=sk // 4)
    if pad_batches == "one":
        mask = mask[:1].contiguous()
    want_y = oracle.masked_softmax_fwd(x, mask, scale)
    dropped, y = [t.cpu() for t in ext.forward_dropout(x.to(DEV), mask.to(DEV), scale, p, seed)]
    util.assert_ulp_close(y, want_y, 2, "y")
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(y, None, None, p, seed)))
    want_dx = oracle.masked_softmax_dropout_bwd(dy, want_y, scale, p, seed)
    got_dx = ext.backward_dropout(dy.to(DEV).clone(), want_y.to(DEV), scale, p, seed).cpu()
    g = oracle.bias_dropout_add(dy, None, None, p, seed)
    util.assert_softmax_bwd_close(got_dx.view(-1, sq, sk), want_dx.view(-1, sq, sk), g.view(-1, sq, sk), want_y.view(-1, sq, sk),
                                  scale, "bwd")
    # p = 0 degenerates to the plain pair
    d0, y0 = ext.forward_dropout(x.to(DEV), mask.to(DEV), scale, 0.0, seed)
    plain = ext.forward(x.to(DEV), mask.to(DEV), scale)
    assert torch.equal(d0, y0) and torch.equal(y0, plain)


# (attn_batches, seq_len, window, zero_block, variant)
BLOCK_CASES = [(4, 2048, None, 512, "plain"), (2, 2048, 700, 256, "plain"), (2, 4096, 1000, 1024, "plain"),
               (1, 8192, 4096, 1024, "plain"), (3, 328, 100, 128, "plain"), (2, 200, None, 64, "plain"),
               (4, 2048, None, 512, "alibi"), (4, 1024, 300, 128, "lengths"), (2, 2048, 700, 256, "dropout"),
               (4, 2048, None, 512, "dropout"), (2, 1001, None, 128, "plain"), (2, 64, None, 8, "plain")]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", BLOCK_CASES, ids=lambda c: f"a{c[0]}_s{c[1]}_w{c[2]}_z{c[3]}_{c[4]}")
def test_block_limited_causal_softmax_writes_only_what_the_caller_reads(case, dtype):
    """The zero_block variants (nhp_causal_softmax_blocks_*, nhp_causal_softmax_dropout_blocks_*): inside the range
    of every row that a block-wise caller reads -- from the block of the first key that the first row of the row's
    block sees to the block of the diagonal -- the oracle's values to the tolerances of the whole-row entry points
    (masked positions exactly +0); outside of it the output buffer keeps the sentinel it was filled with, i.e. is
    not written, and sentinels (NaN patterns) planted there in the inputs of the backward do no harm. Rows on the
    scalar path (seq_len 1001) are written whole."""
    import scaled_upper_triang_masked_softmax_cuda as ext
    from megatron.model.fused_softmax import _written_blocks

    a, s, window, zb, variant = case
    print(f"blocks case {case} {dtype}", flush=True)
    scale, p, seed = 1 / math.sqrt(128), 0.1, 77
    x = util.randn((a, s, s), dtype, seed=s, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=s + 1)
    slopes = lengths = None
    if variant == "alibi":
        slopes = torch.tensor(fb.alibi_slopes(4), dtype=torch.float32)
    if variant == "lengths":
        lengths = torch.tensor([700, 1024], dtype=torch.int32)
    written = _written_blocks(s, zb, window, "cpu") if s % 8 == 0 else torch.ones((s, s), dtype=torch.bool)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    assert bool((written | masked).all())          # everything visible lies inside the written range
    sentinel = 0x7e01                              # a NaN pattern in both 16-bit types
    real_empty = torch.empty_like

    def marked(t, **k):
        out = real_empty(t, **k)
        out.view(torch.int16).fill_(sentinel)
        return out

    def planted(t):                                # the caller's uninitialised memory outside the range
        t = t.clone()
        t.view(torch.int16)[:, ~written] = sentinel
        return t.to(DEV)

    def check_range(got, what, uniform_rows=None):
        got = got.cpu()
        if not bool(written.all()):
            assert bool((util.raw_bits(got)[:, ~written] == sentinel).all()), f"{what}: written outside the range"
        zeros = (written & masked).expand(got.shape).clone()
        if uniform_rows is not None:            # rows that the key lengths leave without a key: 1/s, not zeros
            zeros &= ~uniform_rows[..., None]
        assert int(util.raw_bits(got)[zeros].abs().max() if zeros.any() else 0) == 0, f"{what}: zeros"
        return got

    def inside(got, want):                         # the oracle's values where nothing was written
        return torch.where(written, got, want)

    dl = None if lengths is None else lengths.to(DEV)
    want_y = oracle.causal_softmax_fwd(x, scale, window=window, alibi_slopes=slopes, key_lengths=lengths)
    torch.empty_like = marked
    try:
        if variant == "dropout":
            dropped, y = ext.forward_dropout(x.to(DEV), scale, p, seed, window, zb)
            dropped, y = check_range(dropped, "dropped"), check_range(y, "y")
            util.assert_ulp_close(inside(y, want_y), want_y, 2, "y")
            want_dropped = oracle.bias_dropout_add(inside(y, want_y), None, None, p, seed)
            assert torch.equal(util.raw_bits(dropped)[:, written], util.raw_bits(want_dropped)[:, written])
            dx = check_range(ext.backward_dropout(planted(dy), planted(want_y), scale, p, seed, window, zb), "dx")
            want_dx = oracle.causal_softmax_dropout_bwd(dy, want_y, scale, p, seed, window=window)
            g = oracle.bias_dropout_add(dy, None, None, p, seed)
        else:
            no_key = None if lengths is None else (want_y != 0).sum(-1) == s   # uniform rows of the oracle
            y = check_range(ext.forward(x.to(DEV), scale, window, None if slopes is None else slopes.to(DEV), None, dl,
                                        zb), "y", no_key)
            util.assert_ulp_close(inside(y, want_y), want_y, 2, "y")
            dx = check_range(ext.backward(planted(dy), planted(want_y), scale, window, dl, zb), "dx")
            want_dx = oracle.softmax_bwd(dy, want_y, scale, causal=True, window=window, key_lengths=lengths)
            g = dy
    finally:
        torch.empty_like = real_empty
    dead = want_y == 0                              # masked by the triangle, the window or the key lengths
    util.assert_softmax_bwd_close(inside(dx, want_dx), want_dx, g.masked_fill(dead, 0), want_y, scale, "dx")


def test_block_limited_causal_softmax_at_full_size():
    """[128, 2048, 2048] bf16 (the Pythia-1.4B scores), blocks of 512: inside the written range the forward equals
    the whole-row kernel bit for bit (same launch shape), every row sums to 1, the backward stays within the
    tolerance of the whole-row backward (its row sums are formed by three waves instead of four), and the rest of
    both outputs is left untouched."""
    import scaled_upper_triang_masked_softmax_cuda as ext
    from megatron.model.fused_softmax import _written_blocks

    a, s, zb = 128, 2048, 512
    scale = 1 / math.sqrt(128)
    gen = torch.Generator(device=DEV).manual_seed(3)
    x = (2 * torch.randn((a, s, s), generator=gen, device=DEV)).bfloat16()
    dy = torch.randn((a, s, s), generator=gen, device=DEV).bfloat16()
    written = _written_blocks(s, zb, None, DEV)
    whole = ext.forward(x, scale)
    real_empty = torch.empty_like
    sentinel = 0x7e01

    def marked(t, **k):
        out = real_empty(t, **k)
        out.view(torch.int16).fill_(sentinel)
        return out

    torch.empty_like = marked
    try:
        part = ext.forward(x, scale, None, None, None, None, zb)
    finally:
        torch.empty_like = real_empty
    bits, want = part.view(torch.int16), whole.view(torch.int16)
    assert bool(torch.where(written, bits == want, bits == sentinel).all())
    sums = torch.where(written, part.float(), torch.zeros((), device=DEV)).sum(-1)
    assert (sums - 1).abs().max().item() < 2048 * 2.0 ** -9
    g = dy.clone()
    g.view(torch.int16)[:, ~written] = sentinel           # the caller's uninitialised memory
    got = ext.backward(g, part, scale, None, None, zb)      # in place on g
    ref = ext.backward(dy.clone(), whole, scale)
    gb = got.view(torch.int16)
    assert bool((gb[:, ~written] == sentinel).all())
    diff = torch.where(written, (got.float() - ref.float()).abs(), torch.zeros((), device=DEV))
    bound = torch.where(written, ref.float().abs() * 2.0 ** -7 + 1e-6, torch.ones((), device=DEV))
    assert bool((diff <= bound).all())
    assert int(gb[:, written & (torch.arange(s, device=DEV)[None, :] > torch.arange(s, device=DEV)[:, None])].abs().max()) == 0


# ---------------------------------------------------------------------------
# The padding-mask softmax with bias / AliBi / key lengths inside the kernel, and both softmax kernels with
# those extras and attention dropout at once.
# ---------------------------------------------------------------------------
def abi_masked_ex_fwd(hp, x, mask, scale, slopes=None, bias=None, key_lengths=None, dropout=None):
    """nhp_masked_softmax_ex_fwd, or with dropout=(p, seed) nhp_masked_softmax_ex_dropout_fwd -> (dropped, y)."""
    b, np_, sq, sk = x.shape
    y = torch.empty_like(x)
    m = mask.view(torch.uint8) if mask.dtype == torch.bool else mask
    extras = (None if slopes is None else slopes.data_ptr(), None if bias is None else bias.data_ptr(),
              None if key_lengths is None else key_lengths.data_ptr())
    if dropout is None:
        rc = hp.lib().nhp_masked_softmax_ex_fwd(y.data_ptr(), x.data_ptr(), m.data_ptr(), scale, b, np_, sq, sk, m.size(0),
                                                *extras, hp.dtype_code(x, "t"), None)
        assert rc == 0, hp.lib().nhp_status_string(rc)
        return y
    dropped = torch.empty_like(x)
    rc = hp.lib().nhp_masked_softmax_ex_dropout_fwd(dropped.data_ptr(), y.data_ptr(), x.data_ptr(), m.data_ptr(), scale, b,
                                                    np_, sq, sk, m.size(0), *extras, dropout[0], dropout[1], 0,
                                                    hp.dtype_code(x, "t"), None)
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return dropped, y


# (b, np, sq, sk, extras): every forward geometry of the padding-mask kernel incl. the scalar fallback (sk = 1001, 24);
# "a" AliBi (square scores only), "b" bias tensor, "l" key lengths
MASKED_EX_CASES = [
    (2, 3, 64, 64, "a"), (2, 3, 64, 64, "abl"), (3, 2, 5, 200, "bl"), (2, 2, 512, 512, "al"), (2, 2, 12, 512, "b"),
    (4, 2, 4, 1024, "l"), (2, 4, 1024, 1024, "ab"), (2, 4, 16, 2048, "bl"), (1, 2, 2048, 2048, "abl"), (1, 2, 4, 4096, "bl"),
    (1, 2, 2, 8192, "b"), (2, 2, 6, 1001, "bl"), (2, 2, 1001, 1001, "abl"), (2, 1, 3, 24, "l"), (2, 3, 24, 24, "a"),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("pad_batches", ["one", "each"])
@pytest.mark.parametrize("case", MASKED_EX_CASES, ids=lambda c: "x".join(map(str, c)))
def test_masked_softmax_with_extras_vs_oracle(hotpath, case, pad_batches, dtype):
    """nhp_masked_softmax_ex_fwd against the oracle's composition (eager preparation of scores and mask, then
    the plain padding-mask softmax): 2 ulp, masked keys exactly what the plain kernel leaves there, the scores
    and bias entries of whole chunks of padding keys never read, and the plain entry point's result on the
    prepared operands (bit for bit with key lengths alone, within 1 ulp when AliBi or a bias change the launch shape)."""
    b, np_, sq, sk, extras = case
    print(f"masked ex case {case} {pad_batches} {dtype}", flush=True)
    scale = 1 / math.sqrt(128)
    x = util.randn((b, np_, sq, sk), dtype, seed=sk + sq, std=2.0)
    mask = util.padding_mask(b, sq, sk, seed=sk, lo=sk // 2)
    if sq == sk:
        mask = mask | fb.causal_mask(sk)                  # the decoder's mask: causal and padding
    if pad_batches == "one":
        mask = mask[:1].contiguous()
    slopes = torch.tensor(fb.alibi_slopes(max(np_, 2))[:np_], dtype=torch.float32) if "a" in extras else None
    bias = util.randn((np_, sq, sk), dtype, seed=sk + 7, std=1.5) if "b" in extras else None
    lengths = None
    if "l" in extras:
        lengths = torch.randint(sk // 3, sk + 1, (b,), generator=torch.Generator().manual_seed(sk), dtype=torch.int32)
        lengths[0] = sk - 3                               # a length that cuts a 16-byte chunk
        if b > 1:
            lengths[-1] = 0                               # a sequence without keys: uniform rows
    want = oracle.masked_softmax_fwd(x, mask, scale, slopes, bias, lengths)
    xp, bp = x.clone(), None if bias is None else bias.clone()
    if lengths is not None:
        # whole chunks of padding keys are not read, neither from the scores nor from the bias
        chunk_start = torch.arange(sk) // 8 * 8
        beyond = chunk_start.view(1, 1, 1, sk) >= lengths.view(b, 1, 1, 1)
        xp[beyond.expand_as(xp)] = float("nan")
        if bp is not None:
            bp[(chunk_start.view(1, 1, sk) >= int(lengths.max())).expand_as(bp)] = float("inf")
    dev = lambda t: None if t is None else t.to(DEV)
    got = abi_masked_ex_fwd(hotpath, xp.to(DEV), mask.to(DEV), scale, dev(slopes), dev(bp), dev(lengths)).cpu()
    assert not torch.isnan(got.float()).any()
    util.assert_ulp_close(got, want, 2, "fwd")
    # the same kernel arithmetic as the plain entry point on prepared operands
    xs, ms = oracle.prepared_masked_inputs(x, mask, slopes, bias, lengths)
    plain = util.abi_masked_fwd(hotpath, xs.to(DEV), ms.contiguous().to(DEV), scale).cpu()
    if slopes is None and bias is None:
        assert torch.equal(util.raw_bits(got), util.raw_bits(plain))
    else:
        # per-element extras take a launch shape of their own (one wave per row): another summation order
        util.assert_ulp_close(got, plain, 1, "vs the plain entry point on prepared operands")
        assert torch.equal(util.raw_bits(got) == 0, util.raw_bits(plain) == 0)
    if lengths is not None and b > 1:
        assert torch.equal(got[-1], torch.full_like(got[-1], 1.0 / sk))
    # with dropout on top: the same probabilities, and the oracle's dropout of them
    p, seed = 0.2, 99 + sk
    dropped, y = abi_masked_ex_fwd(hotpath, xp.to(DEV), mask.to(DEV), scale, dev(slopes), dev(bp), dev(lengths), (p, seed))
    assert torch.equal(util.raw_bits(y.cpu()), util.raw_bits(got))
    assert torch.equal(util.raw_bits(dropped.cpu()), util.raw_bits(oracle.bias_dropout_add(got, None, None, p, seed)))


# (batch, heads, seq_len, window, extras, zero_block)
CAUSAL_EX_DROPOUT_CASES = [
    (2, 2, 64, None, "abl", 0), (1, 3, 200, 63, "a", 0), (2, 2, 512, None, "bl", 0), (2, 4, 1024, 100, "al", 0),
    (2, 3, 2048, None, "abl", 0), (1, 2, 4096, 1000, "l", 0), (1, 1, 8192, None, "a", 0), (2, 2, 1001, None, "abl", 0),
    (2, 2, 2048, None, "bl", 512),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("case", CAUSAL_EX_DROPOUT_CASES, ids=lambda c: "_".join(map(str, c)))
def test_causal_softmax_with_extras_and_dropout_vs_oracle(hotpath, case, dtype):
    """nhp_causal_softmax_ex_dropout_fwd/bwd through the extension module: the probabilities are those of the
    entry point without dropout bit for bit (and within 2 ulp of the oracle), `dropped` is the oracle's dropout of
    them, the backward meets the oracle's (dropout backward, then the softmax backward under the same band)."""
    import scaled_upper_triang_masked_softmax_cuda as ext
    from megatron.model.fused_softmax import _written_blocks

    batch, heads, s, window, extras, zb = case
    print(f"causal ex dropout case {case} {dtype}", flush=True)
    a = batch * heads
    scale, p, seed = 1 / math.sqrt(128), 0.1, 555 + s
    x = util.randn((a, s, s), dtype, seed=s + 3, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=s + 4)
    slopes = torch.tensor(fb.alibi_slopes(max(heads, 2))[:heads], dtype=torch.float32) if "a" in extras else None
    bias = util.randn((heads, s, s), dtype, seed=s + 5, std=1.5) if "b" in extras else None
    lengths = torch.tensor([s - 5, s // 3][:batch], dtype=torch.int32) if "l" in extras else None
    dev = lambda t: None if t is None else t.to(DEV)
    want_y = oracle.causal_softmax_fwd(x, scale, window, slopes, bias, lengths)
    written = _written_blocks(s, zb, window, "cpu") if zb else torch.ones((s, s), dtype=torch.bool)
    dropped, y = ext.forward_dropout(x.to(DEV), scale, p, seed, window, zb, dev(slopes), dev(bias), dev(lengths))
    no_drop = ext.forward(x.to(DEV), scale, window, dev(slopes), dev(bias), dev(lengths), zb)
    y, dropped, no_drop = y.cpu(), dropped.cpu(), no_drop.cpu()
    assert torch.equal(util.raw_bits(y)[:, written], util.raw_bits(no_drop)[:, written])
    y = torch.where(written, y, want_y)
    util.assert_ulp_close(y, want_y, 2, "y")
    want_dropped = oracle.bias_dropout_add(y, None, None, p, seed)
    assert torch.equal(util.raw_bits(dropped)[:, written], util.raw_bits(want_dropped)[:, written])
    dead = want_y == 0
    assert int(util.raw_bits(dropped)[:, written][dead[:, written]].abs().max()) == 0
    want_dx = oracle.causal_softmax_dropout_bwd(dy, want_y, scale, p, seed, window=window, key_lengths=lengths)
    got_dx = ext.backward_dropout(dy.to(DEV).clone(), want_y.to(DEV), scale, p, seed, window, zb, dev(lengths)).cpu()
    got_dx = torch.where(written, got_dx, want_dx)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0].expand(a, s, s).clone()
    if lengths is not None:
        masked |= padded_mask(s, lengths, window).repeat_interleave(heads, dim=0)
    assert int(util.raw_bits(got_dx)[masked].abs().max()) == 0
    g = oracle.bias_dropout_add(dy, None, None, p, seed)
    util.assert_softmax_bwd_close(got_dx, want_dx, g.masked_fill(masked, 0), want_y, scale, "bwd")


@pytest.mark.parametrize("fusion", ["upper_triang", "general"])
def test_module_fuses_every_extra_and_dropout_into_one_kernel(fusion, monkeypatch):
    """FusedScaleMaskSoftmax with a bias, AliBi, key lengths and attention dropout together on a fused branch:
    no element-wise torch pass over the scores is left (torch's dropout, add and arange are made to raise), the
    result is the oracle's for the seed the module drew, and the gradients of scores and bias match autograd
    through the torch branch given the same keep mask."""
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T

    dtype, b, np_, s, scale, p = torch.bfloat16, 2, 4, 256, 0.125, 0.25
    slopes = torch.tensor(fb.alibi_slopes(np_), dtype=torch.float32)
    x = util.randn((b, np_, s, s), dtype, seed=1, std=2.0)
    rpe = util.randn((1, np_, s, s), dtype, seed=2)
    dy = util.randn((b, np_, s, s), dtype, seed=3)
    lengths = torch.tensor([s, 100], dtype=torch.int32)
    mask = fb.causal_mask(s, DEV)
    m = FusedScaleMaskSoftmax(False, True, T[fusion], fb.fill_masked_with_dtype_min, True, scale, alibi_slopes=slopes,
                              attention_dropout=p).to(DEV)
    from megatron.model import dropout_rng

    torch.manual_seed(5)
    seed = dropout_rng.next_seed()  # what the module will draw
    torch.manual_seed(5)
    xd, bd, ld = x.to(DEV).requires_grad_(True), rpe.to(DEV).requires_grad_(True), lengths.to(DEV)

    def forbidden(*a, **k):
        raise AssertionError("a torch pass over the scores on the fused branch")

    with monkeypatch.context() as mp:
        mp.setattr(torch.nn.functional, "dropout", forbidden)
        mp.setattr(m, "_add_alibi", forbidden)
        mp.setattr(m, "_mask_with_padding", forbidden)
        out = m(xd, mask, bias=bd, key_lengths=ld)
    out.backward(dy.to(DEV).clone())
    if fusion == "upper_triang":
        want_d, want_y = oracle.causal_softmax_dropout_fwd(x.view(-1, s, s), scale, p, seed, alibi_slopes=slopes,
                                                           bias=rpe[0], key_lengths=lengths)
    else:
        want_d, want_y = oracle.masked_softmax_dropout_fwd(x, mask.cpu(), scale, p, seed, alibi_slopes=slopes,
                                                           bias=rpe[0], key_lengths=lengths)
    want_d, want_y = want_d.view_as(x), want_y.view_as(x)
    keep = oracle.dropout_mask(x.numel(), p, seed).view_as(x)
    got = out.detach().cpu()
    assert int(util.raw_bits(got)[~keep].abs().max()) == 0
    assert (got.float() - want_d.float()).abs().max().item() <= 2.0**-7 * want_d.float().abs().max().item()
    # gradients: float64 autograd of the same function with the same keep mask
    x64, b64 = x.double().requires_grad_(True), rpe.double().requires_grad_(True)
    z = fb.alibi_add((x64 + b64), slopes.double()) * scale
    full = mask.cpu() | (torch.arange(s).view(1, 1, 1, s) >= lengths.view(b, 1, 1, 1))
    probs = torch.softmax(z.masked_fill(full, -10000.0), -1)
    (probs * keep / (1 - p)).backward(dy.double())
    gx, gb = xd.grad.cpu().double(), bd.grad.cpu().double()
    assert (gx - x64.grad).norm().item() <= 2.0**-6 * x64.grad.norm().item()
    assert (gb - b64.grad).norm().item() <= 2.0**-5 * b64.grad.norm().item()
    assert bd.grad.shape == rpe.shape
