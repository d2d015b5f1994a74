"""The drop-in Python surface on the GPU: FusedScaleMaskSoftmax, the autograd
Functions and the fused rotary functions, driven the way GPT-NeoX drives them
(megatron/model/transformer.py:588 and :898-902), checked against the CPU oracle.
Also the relation the reference's own tests rely on: fused ~ torch fallback
(tests/model/test_fused_kernels.py:135,240: mean |diff| <= 1e-3)."""
import math

import pytest
import torch

import oracle
import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"


def mask_func(scores, mask):
    return fb.fill_masked_with_dtype_min(scores, mask)


def make(fusion, dtype, scale):
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax

    return FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, fusion, mask_func, True, scale)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("s", [64, 512, 2048, 4096])
def test_fused_causal_module_forward_backward(dtype, s):
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    b, np_ = 2, 2
    scale = 1 / math.sqrt(128)
    x = util.randn((b, np_, s, s), dtype, seed=s, std=2.0)
    dy = util.randn((b, np_, s, s), dtype, seed=s + 1)
    m = make(T.upper_triang, dtype, scale)
    mask = fb.causal_mask(s, DEV)
    assert m.is_kernel_available(mask, b, np_, s, s)
    xd = x.to(DEV).requires_grad_(True)
    y = m(xd, mask)
    assert y.shape == (b, np_, s, s) and y.dtype == dtype and y.is_contiguous()
    want_y = oracle.causal_softmax_fwd(x.view(-1, s, s), scale).view(b, np_, s, s)
    util.assert_ulp_close(y.detach().cpu(), want_y, 2, "fwd")  # 2 ulp
    g = dy.to(DEV)
    y.backward(g)
    yc = y.detach().cpu()
    want_dx = oracle.softmax_bwd(dy.view(-1, s, s), yc.view(-1, s, s), scale, True).view(b, np_, s, s)
    util.assert_softmax_bwd_close(xd.grad.cpu(), want_dx, dy, yc, scale, "bwd")
    # the backward works in place on the incoming gradient buffer (reference behaviour)
    assert torch.equal(util.raw_bits(g.cpu()), util.raw_bits(xd.grad.cpu()))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("pad_batches", [1, 4])
def test_fused_general_module_forward_backward(dtype, pad_batches):
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    b, np_, sq, sk = 4, 4, 16, 1024
    scale = 0.25
    x = util.randn((b, np_, sq, sk), dtype, seed=3, std=3.0)
    dy = util.randn((b, np_, sq, sk), dtype, seed=4)
    mask = util.padding_mask(pad_batches, sq, sk, seed=5, full_batch=pad_batches - 1 if pad_batches > 1 else None)
    m = make(T.general, dtype, scale)
    assert m.is_kernel_available(mask, b, np_, sq, sk)
    xd = x.to(DEV).requires_grad_(True)
    y = m(xd, mask.to(DEV))
    want_y = oracle.masked_softmax_fwd(x, mask, scale)
    util.assert_ulp_close(y.detach().cpu(), want_y, 2, "fwd")
    y.backward(dy.to(DEV))
    yc = y.detach().cpu()
    util.assert_softmax_bwd_close(xd.grad.cpu(), oracle.softmax_bwd(dy, yc, scale, False), dy, yc, scale, "bwd")


def test_fused_vs_torch_fallback_like_the_reference_tests():
    """The reference compares its fused kernels with its torch path by mean |diff| <= 1e-3."""
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    b, np_, s = 4, 12, 128
    x = util.randn((b, np_, s, s), torch.float16, seed=11, std=1.5).to(DEV)
    causal = fb.causal_mask(s, DEV)
    fused = make(T.upper_triang, torch.float16, None)(x, causal)
    plain = make(T.none, torch.float16, None)(x.clone(), causal)
    assert (fused.float() - plain.float()).abs().mean().item() <= 1e-3
    util.assert_ulp_close(fused.cpu(), plain.cpu(), 2, "causal fused vs torch")
    pad = util.padding_mask(b, s, s, seed=12).to(DEV)
    fused = make(T.general, torch.float16, None)(x, pad)
    plain = make(T.none, torch.float16, None)(x.clone(), pad)
    assert (fused.float() - plain.float()).abs().mean().item() <= 1e-3
    util.assert_ulp_close(fused.cpu(), plain.cpu(), 2, "general fused vs torch")


def test_gate_falls_back_to_torch_ops_on_ineligible_shapes():
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    m = make(T.upper_triang, torch.bfloat16, 0.5)
    s = 30  # sq % 4 != 0
    x = util.randn((2, 2, s, s), torch.bfloat16, seed=1).to(DEV)
    mask = fb.causal_mask(s, DEV)
    assert not m.is_kernel_available(mask, 2, 2, s, s)
    y = m(x, mask)
    want = fb.torch_softmax_fallback(x.cpu(), mask.cpu(), 0.5)
    util.assert_ulp_close(y.cpu(), want, 1, "torch path on GPU vs CPU")


def test_extension_modules_accept_tensor_scale_and_noncontiguous_input():
    import scaled_upper_triang_masked_softmax_cuda as ext

    s = 128
    base = util.randn((4, s, 2 * s), torch.bfloat16, seed=2, std=2.0).to(DEV)
    x = base[..., :s]
    assert not x.is_contiguous()
    scale_t = torch.tensor([0.3])
    y = ext.forward(x, scale_t[0])
    want = oracle.causal_softmax_fwd(x.cpu().contiguous(), 0.3)
    util.assert_ulp_close(y.cpu(), want, 2, "non-contiguous input")
    assert not y.requires_grad
    # a non-contiguous gradient is made contiguous; the returned tensor is that contiguous buffer
    g_base = util.randn((4, s, 2 * s), torch.bfloat16, seed=3).to(DEV)
    g = g_base[..., :s]
    dx = ext.backward(g, y, scale_t[0])
    assert dx.is_contiguous()
    want_dx = oracle.softmax_bwd(g.cpu().contiguous(), y.cpu(), 0.3, True)
    util.assert_softmax_bwd_close(dx.cpu(), want_dx, g.cpu().contiguous(), y.cpu(), 0.3, "bwd")


def test_launches_follow_the_current_stream():
    import scaled_upper_triang_masked_softmax_cuda as ext

    s = 1024
    x = util.randn((8, s, s), torch.bfloat16, seed=5, std=2.0).to(DEV)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        y = ext.forward(x, 0.125)
        done = torch.cuda.Event()
        done.record()
    done.synchronize()
    util.assert_ulp_close(y.cpu(), oracle.causal_softmax_fwd(x.cpu(), 0.125), 2, "side stream")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("rotary_pct", [1.0, 0.25])
def test_fused_rope_cached_like_neox(dtype, rotary_pct):
    """q, k as slices of the fused QKV projection, narrowed for partial rotary,
    rotated with fused_apply_rotary_pos_emb_cached and concatenated with the
    pass-through part (transformer.py:852-914)."""
    from megatron.model.fused_rope import fused_apply_rotary_pos_emb_cached
    from megatron.model.positional_embeddings import RotaryEmbedding

    sq, b, np_, hn = 64, 2, 8, 128
    rot_dim = int(hn * rotary_pct)
    qkv = util.randn((sq, b, np_, 3 * hn), dtype, seed=7)
    qkv_d = qkv.to(DEV).requires_grad_(True)
    q, k, _v = torch.split(qkv_d, hn, dim=3)
    rotary = RotaryEmbedding(rot_dim, sq, base=10000, precision=dtype)
    cos, sin = rotary(_v, seq_len=sq)
    assert cos.device.type == "cuda" and cos.shape == (sq, 1, 1, rot_dim)
    assert rotary(_v, seq_len=sq)[0] is cos  # device copy is made once
    outs = []
    for t in (q, k):
        t_rot, t_pass = (t[..., :rot_dim], t[..., rot_dim:]) if rot_dim < hn else (t, None)
        o = fused_apply_rotary_pos_emb_cached(t_rot, cos, sin)
        outs.append(o if t_pass is None else torch.cat((o, t_pass), dim=-1))
    gq = util.randn((sq, b, np_, hn), dtype, seed=8)
    gk = util.randn((sq, b, np_, hn), dtype, seed=9)
    torch.autograd.backward(outs, [gq.to(DEV), gk.to(DEV)])
    ccos, csin = cos.cpu(), sin.cpu()
    for i, (o, g) in enumerate(zip(outs, (gq, gk))):
        src = qkv[..., i * hn : (i + 1) * hn]
        want = oracle.rope_cached(src, ccos, csin)  # in-kernel pass-through gives the same tensor
        assert torch.equal(util.raw_bits(o.detach().cpu()), util.raw_bits(want))
        want_g = oracle.rope_cached(g, ccos, csin, backward=True)
        got_g = qkv_d.grad[..., i * hn : (i + 1) * hn].cpu()
        assert torch.equal(util.raw_bits(got_g.contiguous()), util.raw_bits(want_g))
    assert (qkv_d.grad[..., 2 * hn :] == 0).all()


def test_fused_rope_full_tensor_pass_through_and_transposed_memory():
    from megatron.model.fused_rope import fused_apply_rotary_pos_emb, fused_apply_rotary_pos_emb_cached
    from megatron.model.positional_embeddings import RotaryEmbedding

    s, b, h, d, d2 = 48, 3, 4, 128, 32
    t = util.randn((s, b, h, d), torch.bfloat16, seed=1)
    rotary = RotaryEmbedding(d2, s, precision=torch.bfloat16)
    td = t.to(DEV).requires_grad_(True)
    cos, sin = rotary(td)
    for transpose in (False, True):
        td.grad = None
        out = fused_apply_rotary_pos_emb_cached(td, cos, sin, transpose)
        assert out.shape == (s, b, h, d)
        assert out.transpose(0, 1).is_contiguous() == transpose
        want = oracle.rope_cached(t, cos.cpu(), sin.cpu())
        assert torch.equal(util.raw_bits(out.detach().cpu().contiguous()), util.raw_bits(want))
        g = util.randn((s, b, h, d), torch.bfloat16, seed=2)
        out.backward(g.to(DEV))
        want_g = oracle.rope_cached(g, cos.cpu(), sin.cpu(), backward=True)
        assert torch.equal(util.raw_bits(td.grad.cpu().contiguous()), util.raw_bits(want_g))
        # the extension's backward lays its result out the same way as the forward
        import fused_rotary_positional_embedding as ext

        raw = ext.backward_cached(g.to(DEV), cos, sin, transpose)
        assert raw.transpose(0, 1).is_contiguous() == transpose
        assert torch.equal(util.raw_bits(raw.cpu().contiguous()), util.raw_bits(want_g))
    # angles variant: freqs = RotaryEmbedding.emb in fp32 on the device
    freqs = rotary.emb.to(DEV)
    assert freqs.dtype == torch.float32 and freqs.shape == (s, 1, 1, d2)
    td.grad = None
    out = fused_apply_rotary_pos_emb(td, freqs)
    want = oracle.rope_freqs(t, rotary.emb)
    bound = 2 * util.ulp_size(t.abs().amax(dim=-1, keepdim=True).expand_as(t).contiguous())
    assert ((out.detach().cpu().float() - want.float()).abs() <= bound).all()  # 2 ulp at input magnitude
    out.backward(torch.ones_like(out))
    assert td.grad.shape == (s, b, h, d)
    assert rotary.get_emb().dtype == torch.bfloat16 and rotary.get_emb().device.type == "cuda"


def test_load_is_idempotent_and_reports_the_native_library():
    import megatron.fused_kernels as fk

    fk.load()
    fk.load()
    fk.load_fused_kernels()
    assert fk._hotpath.lib().nhp_abi_version() == fk._hotpath.ABI_VERSION
    # the shared object is mapped into this process
    assert any("libneox_hotpath.so" in line for line in open("/proc/self/maps"))


def test_baseline_config_c1_whole_tensor_through_the_module():
    """The first configuration of the benchmark set exactly as written: causal forward on scores
    [b=4, h=8, 512, 512] bf16 ~ N(0, 4), scale 1/sqrt(64), seed 0, through FusedScaleMaskSoftmax;
    every element against the oracle (<= 2 ulp), exact zeros above the diagonal, and against the
    reference's torch branch (what that configuration runs on the CPU)."""
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    b, np_, s = 4, 8, 512
    scale = 1 / math.sqrt(64)
    g = torch.Generator().manual_seed(0)
    x = (torch.randn((b, np_, s, s), generator=g) * 2).to(torch.bfloat16)
    mask = fb.causal_mask(s, DEV)
    m = make(T.upper_triang, torch.bfloat16, scale)
    assert m.is_kernel_available(mask, b, np_, s, s)
    y = m(x.to(DEV), mask).cpu()
    assert y.shape == (b, np_, s, s) and y.dtype == torch.bfloat16
    want = oracle.causal_softmax_fwd(x.view(-1, s, s), scale).view(b, np_, s, s)
    util.assert_ulp_close(y, want, 2, "C1 fused vs kernel-semantics oracle")  # 2 bf16 ulp
    above = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
    assert int(util.raw_bits(y)[..., above].abs().max()) == 0, "masked positions must be +0 bit for bit"
    fallback = fb.torch_softmax_fallback(x, mask.cpu(), scale)
    util.assert_ulp_close(y, fallback, 2, "C1 fused vs the torch branch")
    # 0.125 is representable in bf16: the reference kernel's narrowing of the factor changes nothing here
    m_narrow = FusedNarrow(T.upper_triang, torch.bfloat16, scale)
    assert torch.equal(util.raw_bits(m_narrow(x.to(DEV), mask).cpu()), util.raw_bits(y))


def FusedNarrow(fusion, dtype, scale):
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax

    return FusedScaleMaskSoftmax(dtype == torch.float16, dtype == torch.bfloat16, fusion, mask_func, True, scale,
                                 narrow_forward_scale=True)


def _c3_style_scores(shape, seed):
    """fp16 ~ N(0, 9) with 1 % of the entries at +-60, as the padding-mask configuration of the benchmark set."""
    x = util.randn(shape, torch.float16, seed=seed, std=3.0)
    g = torch.Generator().manual_seed(seed + 1)
    hit = torch.rand(shape, generator=g) < 0.01
    sign = torch.where(torch.rand(shape, generator=g) < 0.5, -60.0, 60.0).to(torch.float16)
    return torch.where(hit, sign, x)


@pytest.mark.parametrize("fusion", ["upper_triang", "general"])
def test_narrow_forward_scale_follows_the_reference_kernel(fusion):
    """narrow_forward_scale=True: the forward factor is rounded to the scores' dtype first, as the reference's
    CUDA dispatchers do (scaled_upper_triang_masked_softmax.h:368, scaled_masked_softmax.h:358): within 2 ulp of
    the kernel-semantics oracle called with the narrowed factor, on +-60 outliers where the two factors give
    results up to 3 fp16 ulp apart. Default: within 2 ulp of the oracle with the fp32 factor (= the torch branch).
    The backward uses the fp32 factor in both settings (:467 / :457 take acc_t)."""
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    scale = 1 / math.sqrt(128)
    narrowed = float(torch.tensor(scale).to(torch.float16))
    assert narrowed == 0.08837890625
    if fusion == "upper_triang":
        b, np_, sq, sk = 2, 4, 1024, 1024
        mask = fb.causal_mask(sq, "cpu")
        ref = lambda x, f: oracle.causal_softmax_fwd(x.view(-1, sq, sk), f).view(b, np_, sq, sk)
    else:
        b, np_, sq, sk = 4, 4, 64, 2048
        mask = util.padding_mask(b, sq, sk, seed=9, full_batch=1)
        ref = lambda x, f: oracle.masked_softmax_fwd(x, mask, f)
    x = _c3_style_scores((b, np_, sq, sk), seed=21)
    dy = util.randn((b, np_, sq, sk), torch.float16, seed=23)
    want_full, want_narrow = ref(x, scale), ref(x, narrowed)
    apart = util.ulp_distance(want_full, want_narrow)
    assert int(apart.max()) >= 1 and (apart > 0).float().mean().item() > 0.02, "the inputs must tell the two factors apart"

    results = {}
    for narrow in (False, True):
        m = (FusedNarrow if narrow else make)(getattr(T, fusion), torch.float16, scale)
        xd = x.to(DEV).requires_grad_(True)
        y = m(xd, mask.to(DEV))
        y.backward(dy.to(DEV))
        yc = y.detach().cpu()
        util.assert_ulp_close(yc, want_narrow if narrow else want_full, 2, f"forward, narrow={narrow}")  # 2 fp16 ulp
        want_dx = oracle.softmax_bwd(dy.view(-1, sq, sk), yc.view(-1, sq, sk), scale, fusion == "upper_triang")
        util.assert_softmax_bwd_close(xd.grad.cpu().view(-1, sq, sk), want_dx, dy.view(-1, sq, sk), yc.view(-1, sq, sk),
                                      scale, f"backward with the fp32 factor, narrow={narrow}")
        results[narrow] = yc
    assert not torch.equal(util.raw_bits(results[False]), util.raw_bits(results[True]))


def test_extension_forward_narrow_scale_keyword():
    import scaled_masked_softmax_cuda as masked_ext
    import scaled_upper_triang_masked_softmax_cuda as causal_ext

    scale = 1 / math.sqrt(128)
    narrowed = 0.08837890625
    x = _c3_style_scores((4, 512, 512), seed=31).to(DEV)
    got = causal_ext.forward(x, scale, narrow_scale=True)
    same = causal_ext.forward(x, narrowed)
    assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(same.cpu()))
    xb = x.bfloat16().view(1, 4, 512, 512)
    mask = util.padding_mask(1, 512, 512, seed=3).to(DEV)
    got = masked_ext.forward(xb, mask, scale, narrow_scale=True)
    same = masked_ext.forward(xb, mask, narrowed)  # the bf16 rounding of 1/sqrt(128) is the same number
    assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(same.cpu()))
