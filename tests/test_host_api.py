"""Host-side mirror of the reference API (megatron.model.fused_softmax,
fused_rope, positional_embeddings, megatron.fused_kernels): names, argument
meaning, gating logic and error behaviour. Runs without a GPU."""
import math
import types

import pytest
import torch
import torch.nn.functional as F

import util
from oracle import fallback_semantics as fb


def mask_func(scores, mask):
    return fb.fill_masked_with_dtype_min(scores, mask)


def make(fusion, fp16=True, bf16=False, fp32=True, scale=None):
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax

    return FusedScaleMaskSoftmax(fp16, bf16, fusion, mask_func, fp32, scale)


def test_public_names_exist():
    import megatron.fused_kernels as fk
    import megatron.model.fused_rope as fr
    import megatron.model.fused_softmax as fs
    import megatron.model.positional_embeddings as pe

    for mod, names in ((fs, ["ScaledUpperTriangMaskedSoftmax", "ScaledMaskedSoftmax", "SoftmaxFusionTypes",
                             "FusedScaleMaskSoftmax"]),
                       (fr, ["FusedRoPEFunc", "fused_apply_rotary_pos_emb", "FusedRoPECachedFunc",
                             "fused_apply_rotary_pos_emb_cached"]),
                       (pe, ["RotaryEmbedding", "rotate_half", "apply_rotary_pos_emb", "apply_rotary_pos_emb_torch"]),
                       (fk, ["load", "load_fused_kernels"])):
        for n in names:
            assert hasattr(mod, n), (mod.__name__, n)
    fk.load_fused_kernels()
    import fused_rotary_positional_embedding as rope
    import scaled_masked_softmax_cuda as masked
    import scaled_upper_triang_masked_softmax_cuda as causal

    assert callable(causal.forward) and callable(causal.backward)
    assert callable(masked.forward) and callable(masked.backward) and callable(masked.get_batch_per_block)
    for n in ("forward", "backward", "forward_cached", "backward_cached"):
        assert callable(getattr(rope, n))
    assert [m.value for m in fs.SoftmaxFusionTypes] == [1, 2, 3]


def test_constructor_contract():
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    m = make(T.upper_triang, scale=0.5)
    assert m.input_in_float16 and m.upper_triang_mask_fusion and not m.general_mask_fusion and m.fusion
    m = make(T.general, fp16=False, bf16=True)
    assert m.input_in_float16 and m.general_mask_fusion and m.scale is None
    m = make(T.none, fp16=False, bf16=False)
    assert not m.fusion and not m.input_in_float16
    with pytest.raises(AssertionError, match="softmax should be in fp32 when scaled"):
        make(T.none, fp32=False, scale=2.0)
    with pytest.raises(AssertionError, match="Invalid fusion type"):
        make("upper_triang")


def test_fusion_gate_follows_reference_without_the_2048_cap():
    """fused_softmax.py:148-168: fusion on, 16-bit input, mask given, sk > 16,
    sq % 4 == 0, (b*np) % 4 == 0, plus the batch_per_block divisibility."""
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    mask = torch.zeros(1, 1, 4, 4, dtype=torch.bool)
    causal = make(T.upper_triang, scale=1.0)
    general = make(T.general, scale=1.0)
    assert causal.is_kernel_available(mask, 8, 16, 2048, 2048)
    assert general.is_kernel_available(mask, 16, 32, 1024, 2048)
    assert causal.is_kernel_available(mask, 2, 32, 8192, 8192)  # beyond the reference's 2048 limit
    assert general.is_kernel_available(mask, 2, 2, 8, 4096)
    assert not causal.is_kernel_available(None, 8, 16, 2048, 2048)  # no mask
    assert not causal.is_kernel_available(mask, 8, 16, 16, 16)  # sk must exceed 16
    assert causal.is_kernel_available(mask, 8, 16, 20, 20)
    assert not causal.is_kernel_available(mask, 8, 16, 2046, 2046)  # sq % 4
    assert not causal.is_kernel_available(mask, 1, 6, 64, 64)  # attn_batches % 4
    # batch_per_block on a 64-wide wavefront: sk=32 -> 8 rows per block
    assert causal.get_batch_per_block(32, 32, 1, 4) == 8
    assert not causal.is_kernel_available(mask, 1, 4, 32, 32)  # 4 % 8 != 0
    assert causal.is_kernel_available(mask, 2, 4, 32, 32)
    assert not general.is_kernel_available(mask, 1, 4, 4, 32)  # sq=4, 4 % 8 != 0
    assert general.is_kernel_available(mask, 1, 4, 8, 32)
    assert not make(T.none).is_kernel_available(mask, 8, 16, 2048, 2048)
    assert not make(T.general, fp16=False, bf16=False).is_kernel_available(mask, 8, 16, 2048, 2048)


@pytest.mark.parametrize("dtype,fp16,bf16", [(torch.float16, True, False), (torch.bfloat16, False, True)])
def test_torch_path_matches_reference_fallback_and_kernel_semantics(dtype, fp16, bf16):
    """FusedScaleMaskSoftmax with fusion off runs on CPU: it is the reference's
    fallback, and it agrees with the kernel semantics to 1 ulp on ordinary inputs."""
    import oracle
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    b, np_, s, scale = 2, 4, 64, 1 / math.sqrt(64)
    x = util.randn((b, np_, s, s), dtype, seed=1, std=2.0)
    mask = fb.causal_mask(s)
    m = make(T.none, fp16=fp16, bf16=bf16, scale=scale)
    y = m(x.clone(), mask)
    assert y.dtype == dtype
    assert torch.equal(util.raw_bits(y), util.raw_bits(fb.torch_softmax_fallback(x.clone(), mask, scale)))
    util.assert_ulp_close(y, oracle.causal_softmax_fwd(x.view(-1, s, s), scale).view(b, np_, s, s), 1, "kernel semantics")
    # mask None: plain softmax
    y2 = m(x.clone(), None)
    assert torch.equal(util.raw_bits(y2), util.raw_bits(torch.softmax(x.float() * scale, -1).to(dtype)))
    # native 16-bit softmax when softmax_in_fp32 is off (scale must be None then)
    m16 = make(T.none, fp16=fp16, bf16=bf16, fp32=False)
    assert m16(x.clone(), None).dtype == dtype
    with pytest.raises(AssertionError):
        m(x[0], mask)  # 3-D input


def test_extension_modules_reject_bad_arguments():
    import fused_rotary_positional_embedding as rope
    import scaled_masked_softmax_cuda as masked
    import scaled_upper_triang_masked_softmax_cuda as causal

    x3 = torch.zeros(4, 32, 32, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="expected 3D tensor"):
        causal.forward(x3[0], 1.0)
    with pytest.raises(RuntimeError, match="Only fp16 and bf16 are supported"):
        causal.forward(x3.float(), 1.0)
    with pytest.raises(RuntimeError, match="GPU"):
        causal.forward(x3, 1.0)
    with pytest.raises(RuntimeError, match="expected 3D tensor"):
        causal.backward(x3[0], x3, 1.0)
    x4 = torch.zeros(2, 2, 4, 32, dtype=torch.bfloat16)
    m4 = torch.zeros(2, 1, 4, 32, dtype=torch.bool)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        masked.forward(x4[0], m4, 1.0)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        masked.forward(x4, m4[0], 1.0)
    with pytest.raises(RuntimeError, match="pad_batches"):
        masked.forward(torch.zeros(4, 2, 4, 32, dtype=torch.bfloat16), torch.zeros(3, 1, 4, 32, dtype=torch.bool), 1.0)
    with pytest.raises(RuntimeError, match="query_seq_len > 1"):
        masked.forward(torch.zeros(2, 2, 1, 32, dtype=torch.bfloat16), torch.zeros(2, 1, 1, 32, dtype=torch.bool), 1.0)
    with pytest.raises(RuntimeError, match="Only fp16 and bf16"):
        masked.backward(x4.float(), x4.float(), 1.0)
    t = torch.zeros(8, 2, 2, 16, dtype=torch.bfloat16)
    cos = torch.zeros(8, 1, 1, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="expected 4D tensor"):
        rope.forward_cached(t[0], cos, cos, False)
    with pytest.raises(RuntimeError, match="same sequence length"):
        rope.forward_cached(t, cos[:4], cos[:4], False)
    with pytest.raises(RuntimeError, match="second and third dims"):
        rope.forward_cached(t, cos.expand(8, 2, 1, 16), cos, False)
    with pytest.raises(RuntimeError, match="same last dim"):
        rope.forward_cached(t, cos, cos[..., :8], False)
    with pytest.raises(RuntimeError, match="greater than the cos tensor"):
        rope.forward_cached(t[..., :8], cos, cos, False)
    with pytest.raises(RuntimeError, match="same dtype"):
        rope.backward_cached(t, cos, cos.float(), False)
    with pytest.raises(RuntimeError, match="must be float"):
        rope.forward(t, cos, False)
    with pytest.raises(RuntimeError, match="GPU"):
        rope.forward(t, cos.float(), False)


def test_rotary_embedding_module():
    from megatron.model.positional_embeddings import RotaryEmbedding

    dim, n = 32, 128
    rot = RotaryEmbedding(dim, n, base=10000, precision=torch.bfloat16)
    cos_ref, sin_ref, ang = fb.rotary_tables(dim, n, 10000, torch.bfloat16)
    assert torch.equal(rot.cos_cached, cos_ref) and torch.equal(rot.sin_cached, sin_ref)
    assert torch.equal(rot.emb, ang)
    assert rot.dim == dim and rot.base == 10000 and rot.max_seq_len == n and rot.precision == torch.bfloat16
    # the surviving buffer is cast to `precision`; it is not in the state dict unless asked for
    assert rot.inv_freq.dtype == torch.bfloat16 and rot.inv_freq.shape == (dim // 2,)
    assert "inv_freq" not in rot.state_dict()
    assert "inv_freq" in RotaryEmbedding(dim, n, save_inv_freqs=True).state_dict()
    x = torch.zeros(64, 2, 4, dim)
    cos, sin = rot(x)  # seq_len from x.shape[seq_dim]
    assert cos.shape == (64, 1, 1, dim) and torch.equal(cos, cos_ref[:64])
    cos, sin = rot(x, seq_len=n)
    assert cos.shape == (n, 1, 1, dim)
    cos, sin = rot(x.transpose(0, 1), seq_dim=1)
    assert cos.shape == (64, 1, 1, dim)
    with pytest.raises(AssertionError):
        rot(x, seq_len=n + 1)
    assert RotaryEmbedding(8, 4).cos_cached.dtype == torch.half  # default precision


def test_eager_rotary_functions():
    from megatron.model.positional_embeddings import apply_rotary_pos_emb, apply_rotary_pos_emb_torch, rotate_half

    x = torch.arange(8.0).view(1, 1, 1, 8)
    assert rotate_half(x).flatten().tolist() == [-4, -5, -6, -7, 0, 1, 2, 3]
    s, d = 6, 16
    q = util.randn((s, 2, 2, d), torch.bfloat16, seed=1)
    k = util.randn((s, 2, 2, d), torch.bfloat16, seed=2)
    cos, sin, _ = fb.rotary_tables(d, 16, 10000, torch.bfloat16)
    for fn in (apply_rotary_pos_emb, apply_rotary_pos_emb_torch):
        for offset in (0, 3):
            oq, ok = fn(q, k, cos, sin, offset)
            assert torch.equal(util.raw_bits(oq), util.raw_bits(fb.eager_rotary(q, cos, sin, offset)))
            assert torch.equal(util.raw_bits(ok), util.raw_bits(fb.eager_rotary(k, cos, sin, offset)))


def test_load_fused_kernels_exits_when_not_installed(hotpath, monkeypatch, tmp_path, capsys):
    """Reference behaviour (megatron/fused_kernels/__init__.py:167-181): print a banner and exit()."""
    import megatron.fused_kernels as fk

    monkeypatch.setattr(hotpath, "_lib", None)
    monkeypatch.setattr(hotpath, "LIB_PATH", str(tmp_path / "missing.so"))
    with pytest.raises(SystemExit):
        fk.load_fused_kernels()
    assert "Fused kernels configured but not properly installed" in capsys.readouterr().out


# ---------------------------------------------------------------------------
# the reference's get_norm classes are torch modules that run on any device (megatron/model/norms.py:16,54-119)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_norm_modules_off_the_gpu_follow_the_reference_expressions(dtype):
    from megatron.model import norms

    g = torch.Generator().manual_seed(3)
    x = (torch.randn((3, 5, 32), generator=g) * 2 + 0.5).to(dtype)
    dy = torch.randn((3, 5, 32), generator=g).to(dtype)

    def grads(module, inp):
        inp = inp.clone().requires_grad_(True)
        out = module(inp)
        out.backward(dy.to(out.dtype))
        return out.detach(), inp.grad, [p.grad.clone() for p in module.parameters()]

    # LayerNorm: torch's own class is the reference's
    ours, theirs = norms.LayerNorm(32, eps=1e-5).to(dtype), torch.nn.LayerNorm(32, eps=1e-5).to(dtype)
    with torch.no_grad():
        for p in (ours.weight, theirs.weight):
            p.copy_(torch.linspace(0.5, 1.5, 32))
        for p in (ours.bias, theirs.bias):
            p.copy_(torch.linspace(-1, 1, 32))
    for a, b in zip(grads(ours, x)[:2], grads(theirs, x)[:2]):
        assert a.dtype == b.dtype and torch.equal(a, b)

    # RMSNorm, full and partial, with and without offset: x / (||x[:k]|| / sqrt(k) + eps) * scale [+ offset]
    for p_frac, bias in ((-1.0, False), (0.5, False), (-1.0, True)):
        m = norms.RMSNorm(32, p=p_frac, eps=1e-8, bias=bias).to(dtype)
        with torch.no_grad():
            m.scale.copy_(torch.linspace(0.5, 1.5, 32))
        out, dx, _ = grads(m, x)
        k = 32 if p_frac < 0 else 16
        x64 = x.double().requires_grad_(True)
        rms = x64[..., :k].pow(2).sum(-1, keepdim=True).sqrt() / math.sqrt(k)
        want = m.scale.detach().double() * (x64 / (rms + 1e-8))
        want.backward(dy.double())
        tol = 1e-5 if dtype == torch.float32 else 6e-2
        assert out.dtype == dtype and out.shape == x.shape
        assert (out.double() - want.detach()).abs().max().item() <= tol * max(1.0, want.detach().abs().max().item())
        assert (dx.double() - x64.grad).abs().max().item() <= tol * max(1.0, x64.grad.abs().max().item())
    fused = norms.RMSNorm(32, eps=1e-6, fused_eps=True).to(dtype)
    want = (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).to(dtype)
    assert torch.equal(fused(x).detach(), want)

    # ScaleNorm: x / max(||x||, eps) * g, clamped rows included
    sn = norms.ScaleNorm(32, eps=1e-5).to(dtype)
    with torch.no_grad():
        sn.g.fill_(1.5)
    xs = x.clone()
    xs[0, 0] = 0
    out = sn(xs).detach()
    want = xs.double() / xs.double().norm(dim=-1, keepdim=True).clamp(min=1e-5) * 1.5
    assert out.dtype == dtype and float(out[0, 0].abs().sum()) == 0
    assert (out.double() - want).abs().max().item() <= (1e-5 if dtype == torch.float32 else 3e-2)


# ---------------------------------------------------------------------------
# element-wise and normalisation modules: names, parameters, errors (no GPU needed)
# ---------------------------------------------------------------------------
def test_layer_modules_surface_and_errors():
    import types

    from megatron.model import activations, fused_bias_dropout, norms

    for name in ("bias_gelu", "bias_gelu_back", "GeLUFunction", "bias_gelu_impl"):
        assert hasattr(activations, name)
    for name in ("bias_dropout_add", "get_bias_dropout_add", "bias_dropout_add_fused_train",
                 "bias_dropout_add_fused_inference"):
        assert hasattr(fused_bias_dropout, name)
    # the kernels are the only implementation: CPU tensors are refused, not silently computed elsewhere
    with pytest.raises(RuntimeError, match="GPU"):
        activations.bias_gelu(torch.zeros(8), torch.zeros(2, 8))
    with pytest.raises(RuntimeError, match="GPU"):
        fused_bias_dropout.bias_dropout_add_fused_inference(torch.zeros(2, 8), torch.zeros(8), torch.zeros(2, 8), 0.0)
    with pytest.raises(RuntimeError, match="GPU"):
        fused_bias_dropout.bias_dropout_add(torch.zeros(2, 8), torch.zeros(8), None, 0.1, True)
    ln = norms.LayerNorm(16, eps=1e-5)
    assert sorted(n for n, _ in ln.named_parameters()) == ["bias", "weight"]
    assert ln.weight.shape == (16,) and float(ln.weight.detach().sum()) == 16 and float(ln.bias.detach().abs().sum()) == 0
    assert norms.LayerNorm((16,), elementwise_affine=False).weight is None
    with pytest.raises(NotImplementedError):
        norms.LayerNorm((4, 16))
    rms = norms.RMSNorm(16, eps=1e-8)
    assert [n for n, _ in rms.named_parameters()] == ["scale"] and rms.offset is None
    assert sorted(n for n, _ in norms.RMSNorm(16, bias=True).named_parameters()) == ["offset", "scale"]
    assert norms.RMSNorm(16, p=0.25).partial_size == 4 and norms.RMSNorm(16).partial_size is None
    with pytest.raises(ZeroDivisionError):
        norms.RMSNorm(16, p=0.01)   # int(16 * 0.01) = 0 features: the reference raises the same on its first forward
    sn = norms.ScaleNorm(16, eps=1e-5)
    assert [(n, tuple(p.shape)) for n, p in sn.named_parameters()] == [("g", (1,))] and float(sn.g.detach()) == 1.0
    from megatron.model import fused_layer_norm as fln
    args = types.SimpleNamespace(norm="rmsnorm", rms_norm_epsilon=1e-6, rmsnorm_fusion=True, layernorm_epsilon=1e-5,
                                 layernorm_fusion=True, scalenorm_epsilon=1e-8)
    cls, eps = norms.get_norm(args)
    assert cls is fln.MixedFusedRMSNorm and eps == 1e-6
    fused = cls(8, eps=eps, sequence_parallel=True, apply_rmsnorm_1p=True)
    assert [n for n, _ in fused.named_parameters()] == ["scale"] and fused.scale.sequence_parallel
    assert float(fused.scale.detach().abs().sum()) == 0          # stored as weight - 1
    args.rmsnorm_fusion = False
    assert norms.get_norm(args)[0] is norms.RMSNorm
    args.norm = "layernorm"
    cls, eps = norms.get_norm(args)
    assert cls is fln.MixedFusedLayerNorm and eps == 1e-5
    fl = cls(16, eps=eps)
    assert sorted(n for n, _ in fl.named_parameters()) == ["bias", "weight"] and float(fl.weight.detach().sum()) == 16
    assert fl.normalized_shape == torch.Size([16]) and not fl.weight.sequence_parallel
    args.layernorm_fusion = False
    assert norms.get_norm(args)[0] is norms.LayerNorm
    args.norm = "scalenorm"
    assert norms.get_norm(args) == (norms.ScaleNorm, 1e-8)
    args.norm = "te_rmsnorm"
    with pytest.raises(ValueError):
        norms.get_norm(args)


def test_get_activation_covers_the_reference_settings():
    """get_activation (megatron/model/activations.py:27-66): every setting the reference recognises, the
    gating flag, the onnx_safe / bias_gelu_fusion conflict; the unfused ones against their closed forms."""
    from megatron.model import activations as A

    def pick(name, **kw):
        return A.get_activation(types.SimpleNamespace(activation=name, **kw))

    for name in ("geglu", "reglu", "bilinear", "swiglu", "glu"):
        assert pick(name)[1] is True
    assert pick("gelu", bias_gelu_fusion=True, onnx_safe=False) == (A.bias_gelu_impl, False)
    assert pick("gelu", bias_gelu_fusion=False, onnx_safe=False) == (F.gelu, False)
    assert pick("gelu", bias_gelu_fusion=False, onnx_safe=True) == (A.erf_gelu, False)
    with pytest.raises(ValueError, match="not compatible"):
        pick("gelu", bias_gelu_fusion=True, onnx_safe=True)
    with pytest.raises(ValueError, match="not recognized"):
        pick("tanh")
    x = torch.linspace(-6, 6, 49, dtype=torch.float64)
    for name, want in (("relu", x.clamp(min=0)), ("softsign", x / (1 + x.abs())), ("swish", x / (1 + torch.exp(-x))),
                       ("silu", x / (1 + torch.exp(-x))), ("mish", x * torch.tanh(torch.log1p(torch.exp(x))))):
        func, gated = pick(name)
        assert gated is False and torch.allclose(func(x), want, atol=1e-12), name
    assert torch.allclose(A.erf_gelu(x), x * 0.5 * (1 + torch.erf(x / 1.41421)), atol=1e-12)
    assert torch.allclose(A.erf_gelu(x), F.gelu(x), atol=1e-5)       # 1.41421 is sqrt(2) to 6 digits


def test_sinusoidal_positional_embedding():
    """SinusoidalPositionalEmbedding (megatron/model/positional_embeddings.py:19-35): [1, seq, dim], sines then cosines of
    position * base^(-2j/dim)."""
    from megatron.model.positional_embeddings import SinusoidalPositionalEmbedding

    for precision in (torch.half, torch.bfloat16):
        emb = SinusoidalPositionalEmbedding(16, base=10000, precision=precision)
        out = emb(torch.zeros(2, 7, 16))
        assert out.shape == (1, 7, 16) and emb.inv_freq.shape == (8,)
        assert out.dtype == (torch.bfloat16 if precision == torch.bfloat16 else torch.float32)
        pos = torch.arange(7, dtype=torch.float64)[:, None]
        freq = 10000.0 ** (-torch.arange(0, 16, 2, dtype=torch.float64) / 16)[None, :]
        want = torch.cat((torch.sin(pos * freq), torch.cos(pos * freq)), dim=-1)
        assert torch.allclose(out[0].double(), want, atol=1e-2 if precision == torch.bfloat16 else 1e-6)
        assert emb(torch.zeros(5, 3, 16), seq_dim=0).shape == (1, 5, 16)


def test_core_attention_scaling_and_torch_branch_on_cpu():
    """CoreAttention (the caller of the softmax, megatron/model/transformer.py:417-424, :526-625): the two scaling
    factors, get_fusion_type, and the unfused branch in fp32 against textbook attention in float64."""
    from megatron.model.attention_core import CoreAttention, get_fusion_type
    from megatron.model.fused_softmax import SoftmaxFusionTypes as T

    ns = types.SimpleNamespace
    assert get_fusion_type(ns(scaled_upper_triang_masked_softmax_fusion=True, scaled_masked_softmax_fusion=True)) is T.upper_triang
    assert get_fusion_type(ns(scaled_upper_triang_masked_softmax_fusion=False, scaled_masked_softmax_fusion=True)) is T.general
    assert get_fusion_type(ns(scaled_upper_triang_masked_softmax_fusion=False, scaled_masked_softmax_fusion=False)) is T.none

    def mask_func(scores, mask):
        return fb.fill_masked_with_dtype_min(scores, mask)

    core = CoreAttention(64, 5, False, False, T.none, mask_func, apply_query_key_layer_scaling=True, fold_scale=False)
    assert core.norm_factor == 8 * 5 and core.scale_mask_softmax.scale == 5 and core.scale_mask_softmax.softmax_in_fp32
    assert core.gemm_alpha == 1 / 40
    folded = CoreAttention(64, 5, False, False, T.none, mask_func, apply_query_key_layer_scaling=True)
    assert folded.fold_scale and folded.gemm_alpha == 1.0 and folded.scale_mask_softmax.scale == 5 / 40
    half = CoreAttention(64, 5, True, False, T.none, mask_func, apply_query_key_layer_scaling=True)
    assert not half.fold_scale and half.scale_mask_softmax.scale == 5          # fp16 scores keep the scaled GEMM
    biased = CoreAttention(64, 5, False, True, T.none, mask_func, attention_softmax_in_fp32=True, rpe=lambda a, c: None)
    assert not biased.fold_scale                                               # additive terms come before the scale
    assert CoreAttention(64, 0, False, False, T.none, mask_func, apply_query_key_layer_scaling=True).norm_factor == 8
    assert CoreAttention(64, 5, False, False, T.none, mask_func, use_mup=True).norm_factor == 64
    sq, b, np_, hn = 24, 2, 3, 16
    core = CoreAttention(hn, 3, False, False, T.none, mask_func, apply_query_key_layer_scaling=True)
    q, k, v = (util.randn((sq, b, np_, hn), torch.float32, seed=i) for i in range(3))
    mask = fb.causal_mask(sq, "cpu")
    out = core(q, k, v, mask)
    qd, kd, vd = (t.double().permute(1, 2, 0, 3) for t in (q, k, v))
    scores = (qd @ kd.transpose(-1, -2) / math.sqrt(hn)).masked_fill(mask, float("-inf"))
    want = torch.softmax(scores, -1) @ vd
    assert out.shape == (b, np_, sq, hn) and torch.allclose(out.double(), want, atol=1e-5)
    # with a KV cache the mask is cropped to the keys present
    cached = CoreAttention(hn, 1, False, False, T.none, mask_func, use_cache=True)
    big = fb.causal_mask(sq + 8, "cpu")
    assert torch.allclose(cached(q, k, v, big).double(), want, atol=1e-5)


def test_grouped_query_attention_and_rectangular_scores_on_cpu():
    """CoreAttention with fewer key/value heads than query heads (gqa_project, megatron/model/transformer.py:768-839)
    in fp32 on the CPU against float64 attention over repeated heads, with gradients; and scores that are not
    square (new positions after cached keys) under the causal fusion type, which take the caller's mask."""
    from megatron.model.attention_core import CoreAttention
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes as T

    def mask_func(scores, mask):
        return fb.fill_masked_with_dtype_min(scores, mask)

    sq, b, np_, nkv, hn = 20, 2, 6, 2, 8
    core = CoreAttention(hn, 1, False, False, T.none, mask_func)
    q = util.randn((sq, b, np_, hn), torch.float32, seed=1).requires_grad_(True)
    k = util.randn((sq, b, nkv, hn), torch.float32, seed=2).requires_grad_(True)
    v = util.randn((sq, b, nkv, hn), torch.float32, seed=3).requires_grad_(True)
    mask = fb.causal_mask(sq, "cpu")
    g = util.randn((sq, b, np_ * hn), torch.float32, seed=4)
    out = core(q, k, v, mask, merged_heads=True)
    out.backward(g)
    qd, kd, vd = (t.detach().double().requires_grad_(True) for t in (q, k, v))
    kr, vr = (torch.repeat_interleave(t, np_ // nkv, dim=2) for t in (kd, vd))
    scores = (qd.permute(1, 2, 0, 3) @ kr.permute(1, 2, 3, 0) / math.sqrt(hn)).masked_fill(mask, float("-inf"))
    want = (torch.softmax(scores, -1) @ vr.permute(1, 2, 0, 3)).permute(2, 0, 1, 3).reshape(sq, b, np_ * hn)
    want.backward(g.double())
    assert torch.allclose(out.double(), want, atol=1e-5)
    for got, ref in ((q.grad, qd.grad), (k.grad, kd.grad), (v.grad, vd.grad)):
        assert got.shape == ref.shape and torch.allclose(got.double(), ref, atol=1e-5)
    with pytest.raises(AssertionError):
        core(q, k[:, :, :1].expand(sq, b, 4, hn), v, mask)   # 6 query heads over 4 key heads
    # rows 12..19 of the 20 x 20 causal matrix
    module = FusedScaleMaskSoftmax(False, False, T.upper_triang, mask_func, True, 0.5)
    x = util.randn((b, np_, 8, sq), torch.float32, seed=5)
    rows = mask[..., 12:, :]
    got = module(x, rows)
    ref = torch.softmax((x.double() * 0.5).masked_fill(rows, float("-inf")), -1)
    assert torch.allclose(got.double(), ref, atol=1e-6)


def test_relative_position_bias_buckets_and_values():
    """RelativePositionBias (ParallelRelativePositionBias, megatron/mpu/layers.py:215-381): the T5 bucket function
    pinned by its defining properties and by hand-computed boundaries, the bias by indexing the table directly."""
    from megatron.model.positional_embeddings import ParallelRelativePositionBias, RelativePositionBias

    assert ParallelRelativePositionBias is RelativePositionBias
    torch.manual_seed(0)
    rpe = RelativePositionBias(scale=8.0, causal=True, num_buckets=32, max_distance=128, heads=4)
    assert rpe.weight.shape == (32, 4)
    q_len = k_len = 300
    b = rpe.buckets(q_len, k_len, "cpu")
    assert b.shape == (q_len, k_len) and b.dtype == torch.long
    q, k = torch.meshgrid(torch.arange(q_len), torch.arange(k_len), indexing="ij")
    n = (q - k)
    assert (b[n <= 0] == 0).all()                                   # the present and the future: bucket 0
    assert torch.equal(b[(n > 0) & (n < 16)], n[(n > 0) & (n < 16)])  # one bucket per distance below num_buckets / 2
    assert (b[n >= 128] == 31).all() and b.max() == 31                # everything from max_distance on: the last bucket
    # Toeplitz and monotone in the distance
    first_col = b[:, 0]
    assert all(torch.equal(torch.diagonal(b, -d), first_col[d].expand(q_len - d)) for d in (1, 17, 64, 200))
    assert (first_col[1:] >= first_col[:-1]).all()
    # logarithmic part: bucket 16 + floor(log(n / 16) / log(8) * 16); boundaries by hand: 16 * 8^(j/16)
    for n_val, want in ((16, 16), (18, 16), (19, 17), (22, 18), (32, 21), (45, 23), (46, 24), (64, 26), (91, 29), (127, 31)):
        assert first_col[n_val].item() == want, (n_val, first_col[n_val].item(), want)
    bias = rpe(q_len, k_len)
    assert bias.shape == (1, 4, q_len, k_len)
    for (h, qi, ki) in ((0, 5, 5), (1, 100, 3), (3, 299, 0), (2, 10, 200)):
        assert bias[0, h, qi, ki].item() == pytest.approx(rpe.weight[b[qi, ki], h].item() * 8.0)
    # non-causal: 16 buckets per direction
    both = RelativePositionBias(scale=1.0, causal=False, num_buckets=32, max_distance=128, heads=2)
    bb = both.buckets(200, 200, "cpu")
    assert (bb[n[:200, :200] >= 0] < 16).all() and (bb[n[:200, :200] < 0] >= 16).all()
    assert bb[0, 199].item() == 31 and bb[199, 0].item() == 15 and bb[7, 0].item() == 7 and bb[0, 7].item() == 16 + 7
    # the gradient reaches the table
    bias.sum().backward()
    counts = torch.bincount(b.flatten(), minlength=32).float()
    assert torch.allclose(rpe.weight.grad, (counts * 8.0)[:, None].expand(32, 4))


def test_causal_gemm_blocks_cover_what_is_visible_and_stay_inside_what_the_softmax_writes():
    """The contract between the blocked attention GEMMs and the block-limited causal softmax, by brute force: every
    visible (query, key) pair lies in a row block and in a column block (nothing needed is skipped), and every
    element a block reads lies in the range the kernel writes for that row (nothing uninitialised is read)."""
    from megatron.model import attention_core as ac
    from megatron.model.fused_softmax import _written_blocks

    assert ac.causal_gemm_block(1024) == 0 and ac.causal_gemm_block(2048) == 512 and ac.causal_gemm_block(4096) == 1024
    for s, blk, window in ((64, 16, None), (64, 16, 5), (64, 16, 16), (64, 16, 17), (64, 16, 40), (72, 16, 20),
                           (100, 32, 33), (100, 32, 0), (128, 8, 31), (50, 64, 10), (96, 32, 95), (96, 32, 200)):
        visible = ~fb.causal_mask(s, "cpu", sliding_window_width=window)[0, 0]
        eff = None if window is None or window >= s else window
        written = _written_blocks(s, blk, eff, "cpu")
        rows = torch.zeros((s, s), dtype=torch.bool)
        for r0, r1, c0 in ac._row_blocks(s, blk, eff):
            assert 0 <= c0 <= r0 < r1 <= s and c0 % blk == 0
            rows[r0:r1, c0:r1] = True
        cols = torch.zeros((s, s), dtype=torch.bool)
        for c0, c1, r1 in ac._column_blocks(s, blk, eff):
            assert 0 <= c0 < c1 <= r1 <= s
            cols[c0:r1, c0:c1] = True
        case = (s, blk, window)
        assert bool((rows | ~visible).all()) and bool((cols | ~visible).all()), case     # nothing visible is skipped
        assert bool((written | ~rows).all()) and bool((written | ~cols).all()), case     # nothing unwritten is read
        assert bool((written | ~visible).all()), case
        # and the blocks do save work: no block lies entirely above the diagonal
        assert not bool(rows[0, blk:].any())


def test_attention_mask_producers():
    """get_attn_mask / get_ltor_masks_and_position_ids (megatron/utils.py:67-110): tril of ones, with a window
    triu(diagonal=-width) of it, "< 0.5" -- written out with torch's own tril / triu here."""
    from megatron.model.utils import get_fusion_type
    from megatron.utils import get_attn_mask, get_ltor_masks_and_position_ids

    assert callable(get_fusion_type)
    for s, width in ((1, None), (7, None), (16, 0), (16, 3), (16, 15), (16, 40), (33, 8)):
        ones = torch.tril(torch.ones((1, s, s))).view(1, 1, s, s)
        if width is not None:
            ones = torch.triu(ones, diagonal=-width)
        want = ones < 0.5
        got = get_attn_mask(s, "cpu", width)
        assert got.dtype == torch.bool and got.shape == (1, 1, s, s) and torch.equal(got, want), (s, width)
        assert torch.equal(got, fb.causal_mask(s, "cpu", sliding_window_width=width))
    data = torch.tensor([[5, 0, 7, 0], [1, 2, 3, 4]])
    mask, loss, pos = get_ltor_masks_and_position_ids(data, eod_token=0, eod_mask_loss=True, sliding_window_width=2)
    assert torch.equal(mask, get_attn_mask(4, "cpu", 2))
    assert torch.equal(loss, torch.tensor([[1.0, 0.0, 1.0, 0.0], [1.0, 1.0, 1.0, 1.0]]))
    assert torch.equal(pos, torch.tensor([[0, 1, 2, 3], [0, 1, 2, 3]]))
    assert get_ltor_masks_and_position_ids(data, 0)[1].sum() == 8


def test_dropout_seed_mixing_is_a_bijection_like_spread():
    """The (generator seed, Philox offset) pair is folded into one seed: distinct pairs give distinct, well
    spread values (the device side of dropout_rng is covered by the GPU tests)."""
    from megatron.model.dropout_rng import _mix

    seen = {_mix(s, o) for s in (0, 1, 2, 1234, 2**63 + 5) for o in range(0, 4096, 4)}
    assert len(seen) == 5 * 1024 and all(0 <= v < 2**63 for v in seen)
    assert bin(_mix(0, 0) ^ _mix(0, 4)).count("1") > 16


def test_block_limited_softmax_is_not_part_of_the_public_forward():
    """forward() keeps the reference's call shape plus the two documented extras; the variant that leaves
    blocks of the result unwritten is reachable only through a private method."""
    import inspect

    from megatron.model.fused_softmax import FusedScaleMaskSoftmax

    assert list(inspect.signature(FusedScaleMaskSoftmax.forward).parameters) == ["self", "input", "mask", "bias", "key_lengths"]
    assert hasattr(FusedScaleMaskSoftmax, "_forward_block_limited")


def test_forward_scale_narrowing_helper_and_constructor_flag():
    """The opt-in that reproduces the reference's `const input_t scale` (scaled_upper_triang_masked_softmax.h:368,
    scaled_masked_softmax.h:358): rounding to the scores' dtype, round to nearest even, on the host."""
    from megatron.fused_kernels import _hotpath as hp
    from megatron.model.fused_softmax import FusedScaleMaskSoftmax, SoftmaxFusionTypes

    s128 = 1 / math.sqrt(128)
    for dtype in (torch.float16, torch.bfloat16):
        t = torch.zeros(1, dtype=dtype)
        assert hp.forward_scale(s128, t, False) == s128
        assert hp.forward_scale(s128, t, True) == 0.08837890625
        assert hp.forward_scale(0.125, t, True) == 0.125
        assert hp.forward_scale(torch.tensor([0.3])[0], t, True) == float(torch.tensor(0.3).to(dtype))
    # 1 + 2^-8 is a tie in bf16 (8 significant bits): to even, i.e. down; 1 + 3 * 2^-8 ties up
    bf = torch.zeros(1, dtype=torch.bfloat16)
    assert hp.forward_scale(1 + 2.0**-8, bf, True) == 1.0
    assert hp.forward_scale(1 + 3 * 2.0**-8, bf, True) == 1 + 2.0**-6
    m = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, lambda s, k: s, True, s128)
    assert m.narrow_forward_scale is False
    m = FusedScaleMaskSoftmax(True, False, SoftmaxFusionTypes.none, lambda s, k: s, True, s128, narrow_forward_scale=True)
    assert m.narrow_forward_scale is True
