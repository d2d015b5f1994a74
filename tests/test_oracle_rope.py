"""Pins the CPU oracle of the rotary kernels (oracle/kernel_semantics.c) without
any GPU: identities of a rotation, the eager torch expression it must reproduce
bit for bit, torch.autograd for the backward, and the cache recipe.
"""
import math

import pytest
import torch

import oracle
import util
from oracle import fallback_semantics as fb

DTYPES = [torch.bfloat16, torch.float16, torch.float32]
IDS = ["bf16", "fp16", "fp32"]


def generic_tables(d2, s, dtype, seed=0):
    """Independent angle per (position, feature), so that sin[i] != sin[i + d2/2]."""
    g = torch.Generator().manual_seed(seed)
    ang = (torch.rand((s, 1, 1, d2), generator=g) * 20.0 - 10.0).contiguous()
    return ang.cos().to(dtype).contiguous(), ang.sin().to(dtype).contiguous(), ang


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("d,d2", [(16, 16), (32, 8), (20, 10), (15, 6), (128, 32)])
def test_forward_equals_eager_torch_bit_for_bit(dtype, d, d2):
    """(t*cos) + (rotate_half(t)*sin) evaluated by torch in `dtype` performs the
    same three roundings as the kernels' scalar arithmetic."""
    s, b, h = 7, 2, 3
    t = util.randn((s, b, h, d), dtype, seed=d)
    cos, sin, _ = generic_tables(d2, s, dtype, seed=d2)
    got = oracle.rope_cached(t, cos, sin)
    want = fb.eager_rotary_partial(t, cos, sin)
    assert torch.equal(util.raw_bits(got), util.raw_bits(want))
    # pass-through features are copies
    assert torch.equal(util.raw_bits(got[..., d2:]), util.raw_bits(t[..., d2:]))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("d,d2", [(16, 16), (32, 8), (20, 10)])
def test_backward_equals_autograd_of_eager_bit_for_bit(dtype, d, d2):
    """torch.autograd through the eager expression multiplies the incoming
    gradient by cos and sin in `dtype` and adds the two contributions in `dtype`:
    the same three roundings, and it pairs g[i] with sin[partner]."""
    s, b, h = 5, 2, 2
    t = util.randn((s, b, h, d), dtype, seed=d).requires_grad_(True)
    g = util.randn((s, b, h, d), dtype, seed=d + 1)
    cos, sin, _ = generic_tables(d2, s, dtype, seed=d2 + 3)
    fb.eager_rotary_partial(t, cos, sin).backward(g)
    got = oracle.rope_cached(g, cos, sin, backward=True)
    assert torch.equal(util.raw_bits(got), util.raw_bits(t.grad))


def test_rotation_identities_fp32():
    s, b, h, d = 9, 2, 3, 32
    t = util.randn((s, b, h, d), torch.float32, seed=1)
    cos, sin, ang = fb.rotary_tables(d, s, 10000, torch.float32)
    y = oracle.rope_cached(t, cos.contiguous(), sin.contiguous())
    # position 0: cos = 1, sin = 0 -> identity, exactly
    assert torch.equal(y[0], t[0])
    # each (i, i + d/2) pair is rotated: its norm is preserved
    h2 = d // 2
    n_in = t[..., :h2] ** 2 + t[..., h2:] ** 2
    n_out = y[..., :h2] ** 2 + y[..., h2:] ** 2
    assert torch.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)
    # the rotation angle is position * inv_freq: check one pair explicitly
    p, j = 5, 3
    theta = ang[p, 0, 0, j].item()
    x1, x2 = t[p, 1, 2, j].item(), t[p, 1, 2, j + h2].item()
    assert abs(y[p, 1, 2, j].item() - (x1 * math.cos(theta) - x2 * math.sin(theta))) < 1e-5
    assert abs(y[p, 1, 2, j + h2].item() - (x2 * math.cos(theta) + x1 * math.sin(theta))) < 1e-5
    # backward is the inverse rotation: rope_bwd(rope_fwd(x)) = x
    back = oracle.rope_cached(y, cos.contiguous(), sin.contiguous(), backward=True)
    assert torch.allclose(back, t, rtol=1e-5, atol=1e-5)
    # ... and the adjoint: <rope(x), g> = <x, rope_bwd(g)>
    g = util.randn((s, b, h, d), torch.float32, seed=2)
    gx = oracle.rope_cached(g, cos.contiguous(), sin.contiguous(), backward=True)
    lhs = (y.double() * g.double()).sum().item()
    rhs = (t.double() * gx.double()).sum().item()
    assert abs(lhs - rhs) < 1e-3


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_strides_and_transposed_output(dtype):
    """Inputs are read through their strides (q as a slice of a fused QKV
    projection, a narrowed partial-rotary view); the output is contiguous sbhd,
    or bshd storage viewed as sbhd."""
    s, b, h, hn, d2 = 6, 3, 4, 16, 8
    qkv = util.randn((s, b, h, 3 * hn), dtype, seed=3)
    cos, sin, _ = generic_tables(d2, s, dtype, seed=1)
    for part in range(3):
        view = qkv[..., part * hn : (part + 1) * hn]
        assert not view.is_contiguous()
        want = fb.eager_rotary_partial(view, cos, sin)
        got = oracle.rope_cached(view, cos, sin)
        assert got.is_contiguous() and torch.equal(util.raw_bits(got), util.raw_bits(want))
        got_t = oracle.rope_cached(view, cos, sin, transpose_output=True)
        assert got_t.shape == (s, b, h, hn) and got_t.transpose(0, 1).is_contiguous()
        assert torch.equal(util.raw_bits(got_t.contiguous()), util.raw_bits(want))
        narrow = view[..., :d2]
        got_n = oracle.rope_cached(narrow, cos, sin)
        assert torch.equal(util.raw_bits(got_n), util.raw_bits(fb.eager_rotary(narrow, cos, sin)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_fp32_tables_are_narrowed_first(dtype):
    """cos/sin given in fp32 are converted to the data dtype before use
    (fused_rotary_positional_embedding.h:148-149)."""
    s, b, h, d = 5, 2, 2, 16
    t = util.randn((s, b, h, d), dtype, seed=5)
    cos32, sin32, _ = generic_tables(d, s, torch.float32, seed=2)
    a = oracle.rope_cached(t, cos32, sin32)
    bb = oracle.rope_cached(t, cos32.to(dtype), sin32.to(dtype))
    assert torch.equal(util.raw_bits(a), util.raw_bits(bb))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_freqs_variant_matches_cached_variant(dtype):
    """forward/backward from angles = cached variant with cos/sin of those angles
    evaluated in fp32. libm's cosf/sinf and torch's may differ in the last fp32
    place, which after narrowing can move a table entry by one ulp of `dtype`;
    so the comparison allows 2 ulp at the magnitude of the inputs."""
    s, b, h, d, d2 = 8, 2, 2, 32, 16
    t = util.randn((s, b, h, d), dtype, seed=6)
    _, _, ang = generic_tables(d2, s, torch.float32, seed=4)
    ang = (ang * 300.0).contiguous()  # angles in the thousands of radians
    cos, sin = ang.cos(), ang.sin()
    for backward in (False, True):
        got = oracle.rope_freqs(t, ang, backward=backward)
        want = oracle.rope_cached(t, cos, sin, backward=backward)
        diff = (got.float() - want.float()).abs()
        bound = 2 * util.ulp_size(t.abs().amax(dim=-1, keepdim=True).expand_as(t).contiguous())
        assert (diff <= bound).all()
        assert (util.ulp_distance(got, want) <= 2).float().mean().item() > 0.98


def test_odd_rotary_dim_follows_reference_indexing():
    """d2 = 7: h2 = 3; elements i < 4 pair with i + 3 (negated), the others with i + 3 - 7
    (fused_rotary_positional_embedding.h:54-57)."""
    s, d, d2 = 2, 9, 7
    t = util.randn((s, 1, 1, d), torch.float32, seed=8)
    cos, sin, _ = generic_tables(d2, s, torch.float32, seed=8)
    y = oracle.rope_cached(t, cos, sin)
    for p in range(s):
        for i in range(d2):
            partner = i + 3 if i + 3 < d2 else i + 3 - d2
            r = -t[p, 0, 0, partner] if i + 3 < d2 else t[p, 0, 0, partner]
            want = t[p, 0, 0, i] * cos[p, 0, 0, i] + r * sin[p, 0, 0, i]
            assert y[p, 0, 0, i].item() == want.item()
    assert torch.equal(y[..., d2:], t[..., d2:])


def test_rotary_cache_recipe():
    """RotaryEmbedding._prepare_cache: inv_freq_j = base^(-2j/dim), angle = p * inv_freq,
    the two halves of the feature axis share angles, tables are cast last."""
    dim, s, base = 32, 64, 10000
    cos, sin, ang = fb.rotary_tables(dim, s, base, torch.bfloat16)
    assert cos.shape == (s, 1, 1, dim) and cos.dtype == torch.bfloat16 and ang.dtype == torch.float32
    inv = ang[1, 0, 0, : dim // 2]
    assert inv[0].item() == 1.0
    assert abs(inv[-1].item() - base ** (-(dim - 2) / dim)) < 1e-9
    assert torch.equal(ang[..., : dim // 2], ang[..., dim // 2 :])
    assert (cos[0] == 1).all() and (sin[0] == 0).all()
    p, j = 37, 5
    want = math.cos(p * base ** (-2 * j / dim))
    assert abs(cos[p, 0, 0, j].float().item() - want) <= 2.0**-8
    assert torch.equal(cos, ang.cos().to(torch.bfloat16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_rounding_boundary_marks_cover_every_fp32_perturbation(dtype):
    """util.near_rounding_boundary: an fp32 value that rounds differently to `dtype` after moving
    by up to 2 fp32 spacings must be marked; and only a small share of values is marked."""
    g = torch.Generator().manual_seed(11)
    ang = torch.rand(200000, generator=g, dtype=torch.float64) * 4000.0 - 2000.0
    v = torch.cos(ang)
    marked = util.near_rounding_boundary(v, dtype)
    v32 = v.float()
    base = v32.to(dtype)
    raw = v32.view(torch.int32)
    for k in (-2, -1, 1, 2):
        moved = (raw + k).view(torch.float32)
        flips = moved.to(dtype).view(torch.int16) != base.view(torch.int16)
        assert not (flips & ~marked).any(), k
    assert 0 < float(marked.float().mean()) < (0.002 if dtype == torch.bfloat16 else 0.01)
    # exact midpoints and exact representable values
    one = torch.tensor([1.0], dtype=dtype)
    nxt = (one.view(torch.int16) + 1).view(dtype)
    mid = (one.double() + nxt.double()) / 2
    assert util.near_rounding_boundary(mid, dtype).all()
    assert not util.near_rounding_boundary(one.double(), dtype).any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("backward", [False, True], ids=["fwd", "bwd"])
def test_freqs_tolerance_holds_between_two_host_sincos(dtype, backward):
    """The comparison used for the device's angle variant, exercised on the CPU: the oracle (libm
    sincosf) against the same rotation with tables from torch's cos / sin (another fp32 routine).
    They may differ only on elements marked as resting on a table rounding boundary."""
    s, b, h, d, d2 = 64, 2, 3, 64, 48
    g = torch.Generator().manual_seed(5)
    ang = ((torch.rand((s, 1, 1, d2), generator=g) * 20.0 - 10.0) *
           torch.where(torch.arange(s) % 2 == 0, 1.0, 700.0).view(s, 1, 1, 1)).contiguous()
    t = util.randn((s, b, h, d), dtype, seed=3)
    want = oracle.rope_freqs(t, ang, backward=backward)
    got = oracle.rope_cached(t, ang.cos().to(dtype).contiguous(), ang.sin().to(dtype).contiguous(), backward=backward)
    util.assert_rope_freqs_close(got, want, t, ang, backward, "host sincos pair")
    # a wrong angle index on a handful of elements is caught: swap two positions' angles
    bad_ang = ang.clone()
    bad_ang[[3, 4]] = ang[[4, 3]]
    bad = oracle.rope_cached(t, bad_ang.cos().to(dtype).contiguous(), bad_ang.sin().to(dtype).contiguous(), backward=backward)
    with pytest.raises(AssertionError):
        util.assert_rope_freqs_close(bad, want, t, ang, backward, "swapped angles")
