"""Pins the CPU oracle of the softmax kernels (oracle/kernel_semantics.c) without
any GPU: closed forms, invariants, float64 brute force on tiny inputs and the
torch library routines the reference's own fallback is made of. Each check is
chosen so that a plausible mistake (dropped scale, wrong mask polarity or fill,
off-by-one diagonal, transposed operand, missing term in the Jacobian) fails it.
"""
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


# ---------------------------------------------------------------------------
# storage conversions used by every oracle function
# ---------------------------------------------------------------------------
def test_fp16_conversion_all_patterns():
    lib = oracle.lib()
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    vals = bits.view(torch.float16).float()
    for i in range(0, 65536, 1):
        b = i
        f = lib.oracle_f16_to_float(b)
        want = vals[i].item()
        if math.isnan(want):
            assert math.isnan(f)
        else:
            assert f == want, hex(b)
            assert lib.oracle_float_to_f16(f) == b or (want == 0 and lib.oracle_float_to_f16(f) in (0, 0x8000)), hex(b)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rounding_to_storage_matches_torch(dtype):
    """Round-to-nearest-even including ties, subnormals, overflow and values just
    off a tie, against torch's float32 -> dtype cast."""
    lib = oracle.lib()
    g = torch.Generator().manual_seed(0)
    # random bit patterns cover all exponents; midpoints between neighbours cover ties
    raw = torch.randint(-(2**31), 2**31 - 1, (60000,), generator=g, dtype=torch.int64).to(torch.int32)
    rnd = raw.view(torch.float32)
    grid = torch.randint(0, 65536, (20000,), generator=g).to(torch.int32).to(torch.int16).view(dtype).float()
    nxt = torch.nextafter(grid.to(dtype), torch.tensor(float("inf"), dtype=dtype)).float()
    mid = (grid + nxt) / 2
    cases = torch.cat([rnd, mid, torch.nextafter(mid, mid + 1), torch.nextafter(mid, mid - 1),
                       torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 2.0**-25, 2.0**-24, 3.4e38, -3.4e38])])
    cases = cases[torch.isfinite(cases)]
    want = cases.to(dtype).view(torch.int16).to(torch.int32) & 0xFFFF
    fn = lib.oracle_float_to_bf16 if dtype == torch.bfloat16 else lib.oracle_float_to_f16
    for v, w in zip(cases.tolist(), want.tolist()):
        assert fn(v) == w, (v, hex(w))


# ---------------------------------------------------------------------------
# causal forward
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("s", [1, 2, 3, 8, 17, 33, 64, 100])
def test_causal_fwd_closed_forms(dtype, s):
    # constant input: row q is uniform 1/(q+1) on k <= q, whatever the scale
    x = torch.full((2, s, s), -1.5, dtype=dtype)
    y = oracle.causal_softmax_fwd(x, 0.37)
    q = torch.arange(s)
    want = torch.where(q[None, :] <= q[:, None], (1.0 / (q[:, None] + 1).float()), torch.zeros(())).to(dtype)
    assert torch.equal(util.raw_bits(y[0]), util.raw_bits(want))
    assert torch.equal(util.raw_bits(y[1]), util.raw_bits(want))
    # row 0 is exactly [1, 0, ...] for any input
    x = util.randn((3, s, s), dtype, seed=s, std=5.0)
    y = oracle.causal_softmax_fwd(x, 1.7)
    assert (y[:, 0, 0] == 1).all()
    assert int(util.raw_bits(y[:, 0, 1:]).abs().max() if s > 1 else 0) == 0


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_causal_fwd_two_element_rows_are_logistic(dtype):
    x = util.randn((50, 2, 2), dtype, seed=1, std=3.0)
    scale = 0.8
    y = oracle.causal_softmax_fwd(x, scale)
    d = (x[:, 1, 0].double() - x[:, 1, 1].double()) * float(torch.tensor(scale, dtype=torch.float32))
    want0 = (1 / (1 + torch.exp(-d))).to(dtype)
    want1 = (1 / (1 + torch.exp(d))).to(dtype)
    util.assert_ulp_close(y[:, 1, 0], want0, 1, "logistic 0")
    util.assert_ulp_close(y[:, 1, 1], want1, 1, "logistic 1")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("s", [5, 17, 33, 128, 200])
def test_causal_fwd_vs_float64_and_torch(dtype, s):
    a, scale = 3, 1.0 / math.sqrt(64)
    x = util.randn((a, s, s), dtype, seed=s, std=2.0)
    y = oracle.causal_softmax_fwd(x, scale)
    upper = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
    # masked positions: +0 bit for bit
    assert int(util.raw_bits(y)[:, upper].abs().max()) == 0
    # brute force in float64 (scale as the fp32 value the oracle receives)
    z = x.double() * float(torch.tensor(scale, dtype=torch.float32))
    z = z.masked_fill(upper, float("-inf"))
    want = f64_softmax_rows(z).to(dtype)
    util.assert_ulp_close(y, want, 1, "vs float64")
    # the torch fallback of the reference (fp32 softmax, finfo.min fill)
    ref = fb.torch_softmax_fallback(x.view(1, a, s, s), fb.causal_mask(s), scale).view(a, s, s)
    util.assert_ulp_close(y, ref, 1, "vs torch fallback")
    # rows sum to one within the rounding of their terms
    tol = (2.0**-9 if dtype == torch.bfloat16 else 2.0**-12) * 4
    assert (y.float().sum(-1) - 1).abs().max().item() <= tol * math.sqrt(s) + 1e-6
    # monotone in the logits along a row
    for r in (s - 1, s // 2):
        order = x[0, r, : r + 1].float().argsort()
        assert (y[0, r, : r + 1].float()[order].diff() >= 0).all()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_causal_fwd_shift_invariance_is_exact(dtype):
    """With logits on a 1/4 grid and a power-of-two scale, adding a constant that
    keeps everything representable shifts z exactly, so the outputs are identical."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randint(-40, 40, (2, 48, 48), generator=g).float() / 4).to(dtype)
    a = oracle.causal_softmax_fwd(x, 0.5)
    b = oracle.causal_softmax_fwd((x.float() + 8.0).to(dtype), 0.5)
    assert torch.equal(util.raw_bits(a), util.raw_bits(b))


def test_causal_fwd_scale_is_applied():
    x = util.randn((1, 16, 16), torch.float16, seed=2, std=2.0)
    a = oracle.causal_softmax_fwd(x, 1.0)
    b = oracle.causal_softmax_fwd(x, 0.25)
    c = oracle.causal_softmax_fwd((x.float() * 0.25).to(torch.float16), 1.0)
    assert not torch.equal(a, b)
    util.assert_ulp_close(b, c, 2, "scale")  # x*0.25 is exact in fp16 away from subnormals


# ---------------------------------------------------------------------------
# padding-mask forward
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("sk", [8, 20, 64, 1000, 2048])
def test_masked_fwd_vs_float64_and_fallback(dtype, sk):
    b, np_, sq, scale = 3, 2, 4, 0.3
    x = util.randn((b, np_, sq, sk), dtype, seed=sk, std=3.0)
    mask = util.padding_mask(b, sq, sk, seed=sk, full_batch=2)
    y = oracle.masked_softmax_fwd(x, mask, scale)
    z = x.double() * float(torch.tensor(scale, dtype=torch.float32))
    z = torch.where(mask, torch.tensor(-10000.0, dtype=torch.float64), z)
    util.assert_ulp_close(y, f64_softmax_rows(z).to(dtype), 1, "vs float64")
    # the reference's fallback fills with finfo.min instead of -10000: same result here
    util.assert_ulp_close(y, fb.torch_softmax_fallback(x, mask, scale), 1, "vs torch fallback")
    # fully masked sequence: exactly uniform, i.e. fl(fl32(1/sk))
    uniform = (torch.tensor(1.0, dtype=torch.float32) / sk).to(dtype)
    assert (y[2] == uniform).all()
    # masked keys of partially masked rows: exact zeros
    part = mask.expand(b, np_, sq, sk).clone()
    part[2] = False
    assert int(util.raw_bits(y)[part].abs().max() if part.any() else 0) == 0


def test_masked_fwd_mask_broadcast_and_polarity():
    b, np_, sq, sk = 3, 2, 5, 40
    x = util.randn((b, np_, sq, sk), torch.float16, seed=4, std=2.0)
    m1 = util.padding_mask(1, sq, sk, seed=9)
    shared = oracle.masked_softmax_fwd(x, m1, 0.5)
    expanded = oracle.masked_softmax_fwd(x, m1.expand(b, 1, sq, sk).contiguous(), 0.5)
    assert torch.equal(util.raw_bits(shared), util.raw_bits(expanded))
    # True masks (probability 0), False keeps
    assert (shared[..., m1[0, 0]] == 0).all()
    assert (shared[..., ~m1[0, 0]] > 0).any()
    # per-batch masks are indexed by batch, not by head
    mb = util.padding_mask(b, sq, sk, seed=10)
    per = oracle.masked_softmax_fwd(x, mb, 0.5)
    for bi in range(b):
        one = oracle.masked_softmax_fwd(x[bi : bi + 1], mb[bi : bi + 1], 0.5)
        assert torch.equal(util.raw_bits(per[bi : bi + 1]), util.raw_bits(one))


def test_masked_fwd_only_byte_value_one_masks():
    x = util.randn((1, 1, 2, 16), torch.float16, seed=5)
    m = torch.tensor([0, 1, 2, 255] * 4, dtype=torch.uint8).view(1, 1, 1, 16).expand(1, 1, 2, 16).contiguous()
    y = oracle.masked_softmax_fwd(x, m, 1.0)
    assert (y[..., m[0, 0, 0] == 1] == 0).all()
    assert (y[..., m[0, 0, 0] != 1] > 0).all()


def test_masked_fwd_fill_value_is_minus_10000():
    """With logits near -10000 the fill value shows: a masked key at -10000 ties
    with an unmasked key whose scaled logit is -10000."""
    x = torch.tensor([[-10000.0, -10000.0, 3.0, 3.0]], dtype=torch.float32).to(torch.bfloat16).view(1, 1, 1, 4)
    x = x.expand(1, 1, 2, 4).contiguous()
    m = torch.tensor([False, True, True, True]).view(1, 1, 1, 4).expand(1, 1, 2, 4).contiguous()
    y = oracle.masked_softmax_fwd(x, m, 1.0)
    xs = x[0, 0, 0, 0].float().item()  # -10000 rounded to bf16
    z = torch.tensor([xs, -10000.0, -10000.0, -10000.0], dtype=torch.float64)
    util.assert_ulp_close(y[0, 0, 0], f64_softmax_rows(z).to(torch.bfloat16), 1, "fill")


# ---------------------------------------------------------------------------
# backward
# ---------------------------------------------------------------------------
def jvp_f64(dy, y, scale, causal):
    g = dy.double() * y.double()
    if causal:
        s = y.size(-1)
        keep = ~torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
        g = g * keep
        yy = y.double() * keep
    else:
        yy = y.double()
    return float(torch.tensor(scale, dtype=torch.float32)) * (g - yy * g.sum(-1, keepdim=True))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("causal", [True, False], ids=["causal", "plain"])
@pytest.mark.parametrize("s", [3, 17, 64, 200])
def test_bwd_is_textbook_jacobian_product(dtype, causal, s):
    scale = 0.7
    x = util.randn((2, s, s), dtype, seed=s, std=2.0)
    y = oracle.causal_softmax_fwd(x, scale) if causal else oracle.masked_softmax_fwd(
        x.view(1, 2, s, s), torch.zeros(1, 1, s, s, dtype=torch.bool), scale).view(2, s, s)
    dy = util.randn((2, s, s), dtype, seed=s + 1)
    dx = oracle.softmax_bwd(dy, y, scale, causal)
    want = jvp_f64(dy, y, scale, causal).to(dtype)
    util.assert_softmax_bwd_close(dx, want, dy, y, scale, "vs float64 JVP")
    # the Jacobian annihilates constants: gradient rows sum to ~0
    bound = (dy.float() * y.float()).abs().sum(-1) * scale * 2.0**-7
    assert (dx.float().sum(-1).abs() <= bound + 1e-6).all()
    if causal:
        upper = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
        assert int(util.raw_bits(dx)[:, upper].abs().max() if upper.any() else 0) == 0


def test_bwd_matches_finite_differences_in_float64():
    """d/dx_j of sum_k dy_k softmax(scale*x)_k, rows of a causal matrix."""
    s, scale, eps = 6, 0.9, 1e-6
    g = torch.Generator().manual_seed(0)
    x = torch.randn(s, s, generator=g, dtype=torch.float64)
    dy = torch.randn(s, s, generator=g, dtype=torch.float64)
    upper = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)

    def f(xx):
        z = (xx * scale).masked_fill(upper, float("-inf"))
        return (f64_softmax_rows(z) * dy).sum()

    fd = torch.zeros(s, s, dtype=torch.float64)
    for i in range(s):
        for j in range(i + 1):
            d = torch.zeros(s, s, dtype=torch.float64)
            d[i, j] = eps
            fd[i, j] = (f(x + d) - f(x - d)) / (2 * eps)
    # feed the oracle fp16 copies of y and dy; fp16 rounding bounds the agreement
    y16 = f64_softmax_rows((x * scale).masked_fill(upper, float("-inf"))).to(torch.float16)
    dx = oracle.softmax_bwd(dy.to(torch.float16).view(1, s, s), y16.view(1, s, s), scale, True)[0]
    assert (dx.double() - fd).abs().max().item() < 5e-3
    assert (dx.double() - fd).abs().max().item() < 0.05 * fd.abs().max().item()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bwd_vs_autograd_of_fallback(dtype):
    """Autograd through the reference's torch fallback (fp32) agrees with the fused
    backward up to the rounding of y (the fused backward starts from the rounded y)."""
    b, np_, sq, sk, scale = 2, 2, 4, 64, 0.4
    x = util.randn((b, np_, sq, sk), dtype, seed=7, std=2.0)
    mask = util.padding_mask(b, sq, sk, seed=7)
    dy = util.randn((b, np_, sq, sk), dtype, seed=8)
    xf = x.clone().requires_grad_(True)
    fb.torch_softmax_fallback(xf, mask, scale).backward(dy)
    y = oracle.masked_softmax_fwd(x, mask, scale)
    dx = oracle.softmax_bwd(dy, y, scale, causal=False)
    tol = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    assert (dx.float() - xf.grad.float()).abs().max().item() <= 4 * tol * dy.float().abs().max().item() * scale


def test_bwd_fully_masked_rows_get_nonzero_gradient():
    """The fused backward has no mask argument (scaled_masked_softmax.h:240-335):
    a fully masked row (uniform y) still receives scale*y*(dy - mean dy)."""
    sk = 16
    y = torch.full((1, 1, 2, sk), 1.0 / sk, dtype=torch.float16)
    dy = util.randn((1, 1, 2, sk), torch.float16, seed=1)
    dx = oracle.softmax_bwd(dy, y, 0.5, causal=False)
    want = 0.5 * (1.0 / sk) * (dy.float() - dy.float().mean(-1, keepdim=True))
    assert (dx.float() - want).abs().max().item() < 1e-3
    assert dx.float().abs().max().item() > 0


def test_bwd_in_place_aliasing_allowed():
    dy = util.randn((2, 24, 24), torch.bfloat16, seed=3)
    y = oracle.causal_softmax_fwd(util.randn((2, 24, 24), torch.bfloat16, seed=4), 1.0)
    want = oracle.softmax_bwd(dy, y, 0.3, True)
    work = dy.clone()
    rc = oracle.lib().oracle_softmax_bwd(work.data_ptr(), work.data_ptr(), y.data_ptr(), 0.3, 48, 24, 24, 1, oracle.DT_BF16)
    assert rc == 0 and torch.equal(util.raw_bits(work), util.raw_bits(want))


# ---------------------------------------------------------------------------
# get_batch_per_block
# ---------------------------------------------------------------------------
def test_batch_per_block_table():
    # (sk, value on a 32-wide warp, value on a 64-wide wavefront)
    table = [(1, 256, 256), (8, 32, 32), (17, 8, 8), (32, 8, 8), (33, 8, 4), (64, 8, 4), (100, 8, 4), (128, 8, 4),
             (129, 4, 2), (256, 4, 2), (1000, 4, 2), (2048, 4, 2), (8192, 4, 2)]
    for sk, w32, w64 in table:
        assert oracle.batch_per_block(sk, 32) == w32, sk
        assert oracle.batch_per_block(sk, 64) == w64, sk


# ---------------------------------------------------------------------------
# the reference's forward narrows `scale` to the input dtype; this build does not
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,std,outliers", [(torch.bfloat16, 2.0, False), (torch.float16, 3.0, True)],
                         ids=["bf16_causal_like", "fp16_with_60_outliers"])
def test_scale_narrowing_quirk_is_small_and_quantified(dtype, std, outliers):
    """scaled_upper_triang_masked_softmax.h:368 / scaled_masked_softmax.h:358 take the
    forward scale as `input_t`: 1/sqrt(128) becomes 0.08837890625 in bf16 and fp16
    (relative error 1.07e-4), while the reference's backward and its torch fallback
    use the fp32 value, as this build does everywhere. The effect on a probability is
    about 1.07e-4 * |z - z_max| relative: below one bf16 ulp on N(0,4) scores, and up
    to about 2 fp16 ulp when +-60 outliers stretch z - z_max to ~10."""
    scale = 1.0 / math.sqrt(128.0)
    narrowed = float(torch.tensor(scale).to(dtype))
    assert narrowed == 0.08837890625
    assert abs(narrowed / scale - 1) < 1.1e-4
    x = util.randn((4, 256, 256), dtype, seed=1, std=std)
    if outliers:
        g = torch.Generator().manual_seed(2)
        hit = torch.rand(x.shape, generator=g) < 0.01
        x = torch.where(hit, torch.where(torch.rand(x.shape, generator=g) < 0.5, -60.0, 60.0).to(dtype), x)
    full = oracle.causal_softmax_fwd(x, scale)
    narrow = oracle.causal_softmax_fwd(x, narrowed)
    d = util.ulp_distance(full, narrow)
    assert int(d.max()) <= (1 if dtype == torch.bfloat16 else 3)
    # most elements do not move at all
    assert (d == 0).float().mean().item() > (0.95 if dtype == torch.bfloat16 else 0.6)
