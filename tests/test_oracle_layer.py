"""Pins the oracle's element-wise layer functions (bias + tanh-GeLU forward and
backward, column sums, bias + residual add) without a GPU: float64 closed forms,
torch's library routines, autograd in float64, special values."""
import math

import pytest
import torch
import torch.nn.functional as F

import oracle
import util

DTYPES = [torch.bfloat16, torch.float16, torch.float32]
IDS = ["bf16", "fp16", "fp32"]

C0, C1, C2 = 0.79788456, 0.044715, 0.1070322243  # the literals of megatron/model/activations.py:82,93


def gelu_f64(x):
    x = x.double()
    return x * 0.5 * (1.0 + torch.tanh(C0 * x * (1 + C1 * x * x)))


def inputs(dtype, rows=37, cols=96, seed=0, spread=3.0):
    y = util.randn((rows, cols), dtype, seed=seed, std=spread)
    bias = util.randn((cols,), dtype, seed=seed + 1, std=0.5)
    return y, bias


def test_derivative_constant_is_three_times_the_cubic_coefficient():
    assert abs(C2 - 3 * C1 * C0) < 1e-9
    assert abs(C0 - math.sqrt(2 / math.pi)) < 1e-8


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_gelu_forward_closed_form_and_library(dtype):
    y, bias = inputs(dtype)
    out = oracle.bias_gelu_fwd(y, bias)
    x = bias.double() + y.double()
    x32 = (bias.float() + y.float())
    util.assert_close_ulp_or_noise(out, gelu_f64(x32).to(dtype), 1, util.gelu_noise(x32), "vs float64 closed form")
    # torch's own tanh-GeLU (its constants are the exact sqrt(2/pi) and 0.044715)
    lib = F.gelu(x32, approximate="tanh").to(dtype)
    util.assert_close_ulp_or_noise(out, lib, 1, util.gelu_noise(x32), "vs torch gelu(approximate='tanh')")
    # a dropped cubic term, a wrong sign or a missing 0.5 would be far outside: check a few values by hand
    pts = torch.tensor([[-3.0, -1.0, -0.5, 0.0, 0.5, 1.0, 2.0, 3.0]], dtype=dtype)
    want = torch.tensor([[-0.0036373920, -0.1588080094, -0.1542859972, 0.0, 0.3457140028, 0.8411919906,
                          1.9545976940, 2.9963626080]], dtype=torch.float64)
    got = oracle.bias_gelu_fwd(pts, None).double()
    tol = 2.0 ** (-7 if dtype == torch.bfloat16 else -10 if dtype == torch.float16 else -20)
    assert torch.all((got - want).abs() <= tol * want.abs() + 1e-7)
    del x


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_gelu_forward_special_values(dtype):
    big = 30.0
    v = torch.tensor([[0.0, -0.0, big, -big, float("inf"), float("-inf"), float("nan")]], dtype=dtype)
    out = oracle.bias_gelu_fwd(v, None).float()
    assert out[0, 0] == 0 and out[0, 1] == 0
    assert out[0, 2] == big and out[0, 3] == 0
    assert out[0, 4] == float("inf")
    assert torch.isnan(out[0, 5]) and torch.isnan(out[0, 6])  # -inf * 0 is NaN, as in the reference expression
    # without a bias and with a zero bias: the same bits
    y, _ = inputs(dtype, seed=3)
    assert torch.equal(util.raw_bits(oracle.bias_gelu_fwd(y, None)),
                       util.raw_bits(oracle.bias_gelu_fwd(y, torch.zeros(y.size(-1), dtype=dtype))))


def test_bias_is_added_in_fp32_before_the_activation():
    y, bias = inputs(torch.float32, seed=5)
    assert torch.equal(oracle.bias_gelu_fwd(y, bias), oracle.bias_gelu_fwd(bias + y, None))
    # 16-bit storage: the sum is not rounded to 16 bits first
    y, bias = inputs(torch.bfloat16, seed=6)
    fused = oracle.bias_gelu_fwd(y, bias)
    widened = oracle.bias_gelu_fwd(bias.float() + y.float(), None).to(torch.bfloat16)
    assert torch.equal(util.raw_bits(fused), util.raw_bits(widened))
    eager = oracle.bias_gelu_fwd(bias + y, None)  # x rounded to bf16 first, as eager torch would
    assert not torch.equal(util.raw_bits(fused), util.raw_bits(eager))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_gelu_backward_is_the_derivative_of_forward(dtype):
    y, bias = inputs(dtype, seed=7)
    g = util.randn(y.shape, dtype, seed=9)
    dx = oracle.bias_gelu_bwd(g, y, bias)
    x32 = bias.float() + y.float()
    xd = x32.double().requires_grad_(True)
    gelu_f64(xd).backward(g.double())
    util.assert_close_ulp_or_noise(dx, xd.grad.to(dtype), 1, util.gelu_noise(x32, g), "vs float64 autograd")
    # the reference's own closed form, evaluated in float64
    x = x32.double()
    t = torch.tanh(C0 * x * (1 + C1 * x * x))
    ff = 0.5 * x * ((1 - t * t) * (C0 + C2 * x * x)) + 0.5 * (1 + t)
    util.assert_close_ulp_or_noise(dx, (ff * g.double()).to(dtype), 1, util.gelu_noise(x32, g), "vs float64 formula")
    # torch's library backward of its tanh-GeLU
    xl = x32.clone().requires_grad_(True)
    F.gelu(xl, approximate="tanh").backward(g.float())
    util.assert_close_ulp_or_noise(dx, xl.grad.to(dtype), 1, util.gelu_noise(x32, g), "vs torch gelu backward")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_gelu_backward_special_points(dtype):
    pts = torch.tensor([[0.0, 20.0, -20.0, 1.0]], dtype=dtype)
    g = torch.tensor([[2.0, 3.0, 5.0, 1.0]], dtype=dtype)
    dx = oracle.bias_gelu_bwd(g, pts, None).double()
    assert dx[0, 0] == 1.0           # gelu'(0) = 1/2
    assert dx[0, 1] == 3.0           # identity far to the right
    assert dx[0, 2] == 0.0           # flat far to the left
    assert abs(dx[0, 3] - 1.0829640865) < (2.0**-7 if dtype == torch.bfloat16 else 2.0**-10)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_column_sum(dtype):
    t = util.randn((5, 41, 24), dtype, seed=2)
    got = oracle.column_sum(t)
    want = t.double().sum(dim=(0, 1))
    noise = t.float().abs().sum(dim=(0, 1)) * 16 * util.EPS32
    util.assert_close_ulp_or_noise(got, want.to(dtype), 1, noise, "vs float64")
    ints = torch.randint(-8, 9, (64, 16), generator=torch.Generator().manual_seed(1)).to(dtype)
    assert torch.equal(oracle.column_sum(ints).double(), ints.double().sum(0))
    assert torch.equal(oracle.column_sum(torch.empty((0, 8), dtype=dtype)), torch.zeros(8, dtype=dtype))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_add_residual(dtype):
    x, bias = inputs(dtype, seed=11)
    res = util.randn(x.shape, dtype, seed=12, std=2.0)
    got = oracle.bias_add_residual(x, bias, res)
    # the same three fp32 operations spelled with torch
    want = (res.float() + (x.float() + bias.float())).to(dtype)
    assert torch.equal(util.raw_bits(got), util.raw_bits(want))
    # eager torch in the storage dtype rounds x + bias first: off by at most that rounding
    eager = res + (x + bias)
    if dtype == torch.float32:
        assert torch.equal(got, eager)
    else:
        slack = util.ulp_size(x + bias) / 2 + util.ulp_size(got)
        assert torch.all((got.float() - eager.float()).abs() <= slack)
    assert torch.equal(util.raw_bits(oracle.bias_add_residual(x, None, None)), util.raw_bits(x))
    assert torch.equal(util.raw_bits(oracle.bias_add_residual(x, bias, None)),
                       util.raw_bits((x.float() + bias.float()).to(dtype)))
    assert torch.equal(util.raw_bits(oracle.bias_add_residual(x, None, res)),
                       util.raw_bits((res.float() + x.float()).to(dtype)))


# ---------------------------------------------------------------------------
# LayerNorm / RMSNorm
# ---------------------------------------------------------------------------
def norm_inputs(dtype, rows=23, cols=80, seed=0, pdtype=None):
    pdtype = pdtype or dtype
    x = util.randn((rows, cols), dtype, seed=seed, std=2.0) + 0.5
    gamma = (1 + 0.3 * torch.randn(cols, generator=torch.Generator().manual_seed(seed + 1))).to(pdtype)
    beta = (0.2 * torch.randn(cols, generator=torch.Generator().manual_seed(seed + 2))).to(pdtype)
    dy = util.randn((rows, cols), dtype, seed=seed + 3)
    return x, gamma, beta, dy


def norm_noise(x, gamma, eps_like=util.EPS32):
    """fp32 rounding noise of a normalised, scaled value: a few fp32 spacings of |gamma| * |xhat| ~ |gamma| * 8."""
    g = 1.0 if gamma is None else gamma.float().abs()
    return (g * 64 * eps_like).expand_as(x.float()) if gamma is not None else torch.full_like(x.float(), 64 * eps_like)


@pytest.mark.parametrize("pd", ["same", "fp32"])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_layernorm_forward(dtype, pd):
    pdtype = dtype if pd == "same" else torch.float32
    x, gamma, beta, _ = norm_inputs(dtype, pdtype=pdtype)
    eps = 1e-5
    y, mean, rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    # float64 closed form
    xd = x.double()
    m = xd.mean(-1, keepdim=True)
    v = ((xd - m) ** 2).mean(-1, keepdim=True)
    want = (xd - m) / torch.sqrt(v + eps) * gamma.double() + beta.double()
    util.assert_close_ulp_or_noise(y, want.to(dtype), 1, norm_noise(x, gamma), "vs float64")
    assert torch.allclose(mean.double(), m[:, 0], rtol=0, atol=1e-6)
    assert torch.allclose(rstd.double(), (1 / torch.sqrt(v + eps))[:, 0], rtol=1e-6)
    # torch's library routine on fp32 operands
    lib = F.layer_norm(x.float(), (x.size(-1),), gamma.float(), beta.float(), eps).to(dtype)
    util.assert_close_ulp_or_noise(y, lib, 1, norm_noise(x, gamma), "vs torch layer_norm")
    # without affine terms the rows have zero mean and unit mean square (up to eps and rounding)
    plain, _, _ = oracle.layernorm_fwd(x.float(), None, None, eps)
    assert plain.mean(-1).abs().max() < 1e-6
    assert ((plain ** 2).mean(-1) - 1).abs().max() < 1e-4
    # special cases: a constant row has zero variance -> output beta; biased (not Bessel) variance
    const = torch.full((1, 16), 3.0, dtype=dtype)
    yc, mc, rc = oracle.layernorm_fwd(const, None, None, eps)
    assert yc.abs().max() == 0 and mc[0] == 3.0 and abs(rc[0].item() - eps ** -0.5) < 1e-2
    two = torch.tensor([[1.0, 3.0]], dtype=torch.float32)
    y2, _, r2 = oracle.layernorm_fwd(two, None, None, 0.0)
    assert torch.equal(y2, torch.tensor([[-1.0, 1.0]])) and r2[0] == 1.0


@pytest.mark.parametrize("pd", ["same", "fp32"])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_layernorm_backward_is_the_adjoint(dtype, pd):
    pdtype = dtype if pd == "same" else torch.float32
    x, gamma, beta, dy = norm_inputs(dtype, seed=4, pdtype=pdtype)
    eps = 1e-5
    _, mean, rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    dx, dg, db = oracle.layernorm_bwd(dy, x, mean, rstd, gamma)
    xd = x.double().requires_grad_(True)
    gd = gamma.double().requires_grad_(True)
    bd = beta.double().requires_grad_(True)
    F.layer_norm(xd, (x.size(-1),), gd, bd, eps).backward(dy.double())
    scale = (dy.float().abs() * gamma.float().abs()).sum(-1, keepdim=True) * rstd[:, None] * 16 * util.EPS32
    util.assert_close_ulp_or_noise(dx, xd.grad.to(dtype), 1, scale.expand_as(dx.float()) * 8, "dx vs float64 autograd")
    col_noise = dy.float().abs().sum(0) * 64 * util.EPS32 * 8
    util.assert_close_ulp_or_noise(dg, gd.grad.to(pdtype), 1, col_noise, "dgamma")
    util.assert_close_ulp_or_noise(db, bd.grad.to(pdtype), 1, col_noise, "dbeta")
    # the gradient is orthogonal to the two directions LayerNorm removes: constants and xhat
    x32, g32, b32, dy32 = norm_inputs(torch.float32, seed=4)
    _, m32, r32 = oracle.layernorm_fwd(x32, g32, b32, eps)
    dx32, _, _ = oracle.layernorm_bwd(dy32, x32, m32, r32, g32)
    xhat = (x32 - m32[:, None]) * r32[:, None]
    assert dx32.sum(-1).abs().max() < 1e-4
    assert (dx32 * xhat).sum(-1).abs().max() < 1e-3


@pytest.mark.parametrize("pd", ["same", "fp32"])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_layernorm_pair_is_the_sum_of_two_layernorms(dtype, pd):
    """Two LayerNorms of one input: outputs are the two single outputs, dx is the gradient of
    y1.dy1 + y2.dy2 (float64 autograd through torch's layer_norm), rounded once."""
    pdtype = dtype if pd == "same" else torch.float32
    x, gamma1, beta1, dy1 = norm_inputs(dtype, seed=21, pdtype=pdtype)
    _, gamma2, beta2, dy2 = norm_inputs(dtype, seed=22, pdtype=pdtype)
    eps = 1e-5
    y1, y2, mean, rstd = oracle.layernorm_pair_fwd(x, gamma1, beta1, gamma2, beta2, eps)
    s1, m1, r1 = oracle.layernorm_fwd(x, gamma1, beta1, eps)
    s2, _, _ = oracle.layernorm_fwd(x, gamma2, beta2, eps)
    assert torch.equal(y1, s1) and torch.equal(y2, s2) and torch.equal(mean, m1) and torch.equal(rstd, r1)
    dx, dg1, db1, dg2, db2 = oracle.layernorm_pair_bwd(dy1, dy2, x, mean, rstd, gamma1, gamma2)
    xd = x.double().requires_grad_(True)
    params = [t.double().requires_grad_(True) for t in (gamma1, beta1, gamma2, beta2)]
    n = (x.size(-1),)
    loss = (F.layer_norm(xd, n, params[0], params[1], eps) * dy1.double()).sum() + \
           (F.layer_norm(xd, n, params[2], params[3], eps) * dy2.double()).sum()
    loss.backward()
    scale = ((dy1.float().abs() * gamma1.float().abs() + dy2.float().abs() * gamma2.float().abs()).sum(-1, keepdim=True)
             * rstd[:, None] * 128 * util.EPS32)
    util.assert_close_ulp_or_noise(dx, xd.grad.to(dtype), 1, scale.expand_as(dx.float()), "dx vs float64 autograd")
    # parameter gradients are those of the single norms, bit for bit
    _, w1, c1 = oracle.layernorm_bwd(dy1, x, mean, rstd, gamma1)
    _, w2, c2 = oracle.layernorm_bwd(dy2, x, mean, rstd, gamma2)
    assert torch.equal(dg1, w1) and torch.equal(db1, c1) and torch.equal(dg2, w2) and torch.equal(db2, c2)
    for got, want in zip((dg1, db1, dg2, db2), params):
        col = (dy1.float().abs() + dy2.float().abs()).sum(0) * 512 * util.EPS32
        util.assert_close_ulp_or_noise(got, want.grad.to(pdtype), 1, col, "parameter gradient vs float64")
    # a zero second gradient reduces it to the single backward, bit for bit; and swapping the two norms changes nothing
    zero = torch.zeros_like(dy2)
    single, _, _ = oracle.layernorm_bwd(dy1, x, mean, rstd, gamma1)
    assert torch.equal(oracle.layernorm_pair_bwd(dy1, zero, x, mean, rstd, gamma1, gamma2)[0], single)
    swapped = oracle.layernorm_pair_bwd(dy2, dy1, x, mean, rstd, gamma2, gamma1)[0]
    util.assert_close_ulp_or_noise(swapped, dx, 1, scale.expand_as(dx.float()), "order of the two norms")
    # one rounding: in fp32 the pair's dx equals the sum of the two single dx up to fp32 noise, and for 16-bit data it
    # is at least as close to the float64 gradient as the rounded sum of two rounded gradients
    d1, _, _ = oracle.layernorm_bwd(dy1, x, mean, rstd, gamma1)
    d2, _, _ = oracle.layernorm_bwd(dy2, x, mean, rstd, gamma2)
    two_step = (d1 + d2)
    err_pair = (dx.double() - xd.grad).abs().mean()
    err_two = (two_step.double() - xd.grad).abs().mean()
    assert err_pair <= err_two * 1.001 + 1e-12


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_forward(dtype, mode):
    x, scale, offset, _ = norm_inputs(dtype, seed=8)
    eps = 1e-6 if mode == 0 else 1e-3  # an eps large enough to tell the two placements apart
    y, inv = oracle.rmsnorm_fwd(x, scale, offset, eps, mode)
    xd = x.double()
    ms = (xd ** 2).mean(-1, keepdim=True)
    inv64 = 1 / (torch.sqrt(ms) + eps) if mode == 1 else 1 / torch.sqrt(ms + eps)
    want = scale.double() * (xd * inv64) + offset.double()
    util.assert_close_ulp_or_noise(y, want.to(dtype), 1, norm_noise(x, scale), "vs float64")
    assert torch.allclose(inv.double(), inv64[:, 0], rtol=1e-6)
    other, _ = oracle.rmsnorm_fwd(x.float(), scale.float(), offset.float(), eps, 1 - mode)
    mine, _ = oracle.rmsnorm_fwd(x.float(), scale.float(), offset.float(), eps, mode)
    assert not torch.equal(other, mine)
    if mode == 1:
        # the reference's Python class, spelled with the same torch calls in fp32
        x32 = x.float()
        norm_x = x32.norm(2, dim=-1, keepdim=True)
        rms_x = norm_x * x.size(-1) ** (-1.0 / 2)
        ref = scale.float() * (x32 / (rms_x + eps)) + offset.float()
        util.assert_close_ulp_or_noise(y, ref.to(dtype), 1, norm_noise(x, scale), "vs the class's expression in fp32")
    else:
        ref = F.rms_norm(x.float(), (x.size(-1),), scale.float(), eps) + offset.float()
        util.assert_close_ulp_or_noise(y, ref.to(dtype), 1, norm_noise(x, scale), "vs torch rms_norm")
    # unit scale, no offset, eps 0: rows of unit mean square; an all-zero row stays zero with eps > 0
    plain, _ = oracle.rmsnorm_fwd(x.float(), None, None, 0.0, mode)
    assert ((plain ** 2).mean(-1) - 1).abs().max() < 1e-5
    zero, zinv = oracle.rmsnorm_fwd(torch.zeros((1, 8), dtype=dtype), None, None, 1e-3, mode)
    assert zero.abs().max() == 0 and torch.isfinite(zinv).all()


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_rmsnorm_backward_is_the_adjoint(dtype, mode):
    x, scale, offset, dy = norm_inputs(dtype, seed=12)
    eps = 1e-6 if mode == 0 else 1e-2
    _, inv = oracle.rmsnorm_fwd(x, scale, offset, eps, mode)
    dx, ds, do = oracle.rmsnorm_bwd(dy, x, inv, scale, eps, mode)
    xd = x.double().requires_grad_(True)
    sd = scale.double().requires_grad_(True)
    od = offset.double().requires_grad_(True)
    ms = (xd ** 2).mean(-1, keepdim=True)
    inv64 = 1 / (torch.sqrt(ms) + eps) if mode == 1 else 1 / torch.sqrt(ms + eps)
    (sd * (xd * inv64) + od).backward(dy.double())
    noise = (dy.float().abs() * scale.float().abs()).sum(-1, keepdim=True) * inv[:, None] * 128 * util.EPS32
    util.assert_close_ulp_or_noise(dx, xd.grad.to(dtype), 1, noise.expand_as(dx.float()), "dx vs float64 autograd")
    col_noise = dy.float().abs().sum(0) * 512 * util.EPS32
    util.assert_close_ulp_or_noise(ds, sd.grad.to(dtype), 1, col_noise, "dscale")
    util.assert_close_ulp_or_noise(do, od.grad.to(dtype), 1, col_noise, "doffset")
    # an all-zero row: finite gradient, the projection term vanishes
    z = torch.zeros((1, 8), dtype=torch.float32)
    g = torch.ones((1, 8), dtype=torch.float32)
    _, zi = oracle.rmsnorm_fwd(z, None, None, 1e-3, mode)
    dz, _, _ = oracle.rmsnorm_bwd(g, z, zi, None, 1e-3, mode)
    assert torch.isfinite(dz).all() and torch.allclose(dz, g * zi[0])


@pytest.mark.parametrize("frac", [0.5, 0.3, 1.0, 0.01])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_partial_rmsnorm_is_the_class_expression(dtype, frac):
    """RMSNorm with 0 <= p <= 1 (megatron/model/norms.py:87-94): the statistic comes from the first
    int(dim * p) columns, every column is divided by it. Spelled here with the class's own torch
    calls in fp32 and in float64; the backward against float64 autograd of the same expression."""
    x, scale, offset, dy = norm_inputs(dtype, seed=21)
    d = x.size(-1)
    part = max(int(d * frac), 1)
    eps = 1e-3
    y, inv = oracle.rmsnorm_fwd(x, scale, offset, eps, 1, stat_cols=part)

    def class_forward(xx, sc, of):
        partial_x, _ = torch.split(xx, [part, d - part], dim=-1)
        norm_x = partial_x.norm(2, dim=-1, keepdim=True)
        rms_x = norm_x * part ** (-1.0 / 2)
        return sc * (xx / (rms_x + eps)) + of

    util.assert_close_ulp_or_noise(y, class_forward(x.float(), scale.float(), offset.float()).to(dtype), 1,
                                   norm_noise(x, scale) * (d / part) ** 0.5, "vs the class's expression in fp32")
    xd = x.double().requires_grad_(True)
    sd = scale.double().requires_grad_(True)
    od = offset.double().requires_grad_(True)
    out = class_forward(xd, sd, od)
    util.assert_close_ulp_or_noise(y, out.detach().to(dtype), 1, norm_noise(x, scale) * (d / part) ** 0.5, "vs float64")
    out.backward(dy.double())
    dx, ds, do = oracle.rmsnorm_bwd(dy, x, inv, scale, eps, 1, stat_cols=part)
    noise = (dy.float().abs() * scale.float().abs() * x.float().abs()).sum(-1, keepdim=True) * inv[:, None] ** 2 \
        * x.float().abs().amax(-1, keepdim=True) * 256 * util.EPS32 * (d / part) \
        + (dy.float().abs() * scale.float().abs()).amax(-1, keepdim=True) * inv[:, None] * 16 * util.EPS32
    util.assert_close_ulp_or_noise(dx, xd.grad.to(dtype), 1, noise.expand_as(dx.float()), "dx vs float64 autograd")
    col_noise = (dy.float().abs() * x.float().abs() * inv[:, None]).sum(0) * 64 * util.EPS32 + dy.float().abs().sum(0) * 64 * util.EPS32
    util.assert_close_ulp_or_noise(ds, sd.grad.to(dtype), 1, col_noise, "dscale")
    util.assert_close_ulp_or_noise(do, od.grad.to(dtype), 1, col_noise, "doffset")
    if part == d:
        full, finv = oracle.rmsnorm_fwd(x, scale, offset, eps, 1)
        assert torch.equal(full, y) and torch.equal(finv, inv)
    else:
        # columns outside the statistic only see the first term of the gradient
        x32, s32, o32, dy32 = norm_inputs(torch.float32, seed=21)
        _, i32 = oracle.rmsnorm_fwd(x32, s32, o32, eps, 1, stat_cols=part)
        dx32, _, _ = oracle.rmsnorm_bwd(dy32, x32, i32, s32, eps, 1, stat_cols=part)
        assert torch.equal(dx32[:, part:], i32[:, None] * (dy32 * s32)[:, part:])
    # the other epsilon placement takes the same statistic columns
    y0, inv0 = oracle.rmsnorm_fwd(x.float(), None, None, 1e-6, 0, stat_cols=part)
    want0 = x.double() / torch.sqrt((x.double()[:, :part] ** 2).mean(-1, keepdim=True) + 1e-6)
    assert torch.allclose(y0.double(), want0, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_scalenorm_is_the_class_expression(dtype):
    """ScaleNorm.forward (megatron/model/norms.py:117-119): x / clamp(||x||, min=eps) * g with a scalar g;
    a row whose norm is below eps is divided by eps and its norm has no gradient."""
    x, _, _, dy = norm_inputs(dtype, seed=31)
    x = x.clone()
    x[3] = x[3] * 1e-4          # clamped row (norm below eps)
    x[5] = 0                    # all-zero row
    eps = 1e-2
    g = torch.tensor([1.7], dtype=torch.float32)
    cols = x.size(-1)
    gvec = g.to(dtype).expand(cols).contiguous()
    y, inv = oracle.rmsnorm_fwd(x, gvec, None, eps, 2)

    def class_forward(xx, gg):
        n = torch.norm(xx, dim=-1, keepdim=True).clamp(min=eps)
        return xx / n * gg

    ref32 = class_forward(x.float(), g.to(dtype).float())
    noise = x.float().abs() * inv[:, None] * 1.7 * 8 * util.EPS32
    util.assert_close_ulp_or_noise(y, ref32.to(dtype), 1, noise, "vs the class's expression in fp32")
    assert torch.allclose(inv[3], torch.tensor(1 / eps)) and torch.allclose(inv[5], torch.tensor(1 / eps))
    assert y[5].abs().max() == 0
    xd = x.double().requires_grad_(True)
    gd = g.to(dtype).double().requires_grad_(True)
    class_forward(xd, gd).backward(dy.double())
    dx, ds, _ = oracle.rmsnorm_bwd(dy, x, inv, gvec, eps, 2)
    bnoise = (dy.float().abs() * 1.7).sum(-1, keepdim=True) * inv[:, None] * 128 * util.EPS32
    util.assert_close_ulp_or_noise(dx, xd.grad.to(dtype), 1, bnoise.expand_as(dx.float()), "dx vs float64 autograd")
    # the scalar's gradient is the sum of the per-column gradients
    dg = ds.double().sum()
    tol = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1e-2}[dtype]  # per-column sums are rounded to dtype
    assert abs(dg - gd.grad[0]) <= tol * (dy.double().abs() * (x.double() * inv[:, None].double()).abs()).sum()
    # unclamped rows come out with unit norm times g
    y32, _ = oracle.rmsnorm_fwd(x.float(), g.expand(cols).contiguous(), None, eps, 2)
    norms = y32.norm(dim=-1)
    keep = torch.ones(x.size(0), dtype=torch.bool)
    keep[3] = keep[5] = False
    assert (norms[keep] - 1.7).abs().max() < 1e-5


# ---------------------------------------------------------------------------
# gated activations
# ---------------------------------------------------------------------------
def swish(x):
    return x * torch.sigmoid(1.0 * x)  # megatron/model/activations.py:128-130 with beta = 1


GATE_FUNCS = {"swiglu": swish, "geglu": F.gelu, "reglu": F.relu, "glu": torch.sigmoid, "bilinear": lambda x: x}


def reference_gated(inp, bias, act):
    """Gated_Activation.forward (megatron/model/transformer.py:192-206) with torch calls."""
    x, gate = inp.chunk(2, dim=-1)
    if bias is not None:
        b1, b2 = bias.chunk(2, dim=-1)
        x = x + b1
        gate = gate + b2
    return GATE_FUNCS[act](gate) * x


@pytest.mark.parametrize("act", sorted(GATE_FUNCS))
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_gated_activation_forward(dtype, act):
    inp = util.randn((9, 2 * 40), dtype, seed=3, std=2.5)
    bias = util.randn((2 * 40,), dtype, seed=4, std=0.5)
    for b in (None, bias):
        out = oracle.gated_act_fwd(inp, act, b)
        want64 = reference_gated(inp.double(), None if b is None else b.double(), act)
        noise = util.gated_noise(inp, b, act, want64)
        util.assert_close_ulp_or_noise(out, want64.to(dtype), 1, noise, f"{act} vs float64")
        want32 = reference_gated(inp.float(), None if b is None else b.float(), act)
        util.assert_close_ulp_or_noise(out, want32.to(dtype), 1, noise, f"{act} vs torch fp32")
    # which half gates which: swapping the halves changes the result (except for the symmetric bilinear case)
    swapped = torch.cat(inp.chunk(2, -1)[::-1], -1)
    same = torch.equal(util.raw_bits(oracle.gated_act_fwd(swapped, act)), util.raw_bits(oracle.gated_act_fwd(inp, act)))
    assert same == (act == "bilinear")
    # known values: act(0) * x, and a closed form per activation at gate = 1, x = 2
    one = torch.tensor([[2.0, 1.0]], dtype=torch.float32)
    expect = {"swiglu": 2 / (1 + math.exp(-1.0)), "geglu": 2 * 0.5 * (1 + math.erf(2 ** -0.5)), "reglu": 2.0,
              "glu": 2 / (1 + math.exp(-1.0)), "bilinear": 2.0}[act]
    assert abs(oracle.gated_act_fwd(one, act).item() - expect) < 1e-6


@pytest.mark.parametrize("act", sorted(GATE_FUNCS))
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_gated_activation_backward_is_the_adjoint(dtype, act):
    inp = util.randn((7, 2 * 24), dtype, seed=5, std=2.0)
    bias = util.randn((2 * 24,), dtype, seed=6, std=0.5)
    dy = util.randn((7, 24), dtype, seed=7)
    din = oracle.gated_act_bwd(dy, inp, act, bias)
    x64 = inp.double().requires_grad_(True)
    reference_gated(x64, bias.double(), act).backward(dy.double())
    noise = util.gated_noise(inp, bias, act, x64.grad, dy)
    util.assert_close_ulp_or_noise(din, x64.grad.to(dtype), 1, noise, f"{act} vs float64 autograd")
    x32 = inp.float().requires_grad_(True)
    reference_gated(x32, bias.float(), act).backward(dy.float())
    util.assert_close_ulp_or_noise(din, x32.grad.to(dtype), 1, noise, f"{act} vs fp32 autograd")


# ---------------------------------------------------------------------------
# dropout
# ---------------------------------------------------------------------------
PHILOX_KAT = [  # known-answer vectors published with Random123 (philox4x32, 10 rounds)
    ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


def test_philox_known_answers(hotpath):
    import ctypes

    for counter, key, want in PHILOX_KAT:
        assert oracle.philox4x32_10(counter, key) == want
        out = (ctypes.c_uint32 * 4)()
        hotpath.lib().nhp_philox4x32_10((ctypes.c_uint32 * 4)(*counter), (ctypes.c_uint32 * 2)(*key), out)
        assert list(out) == want


def test_dropout_mask_is_bernoulli_and_keyed():
    n = 1 << 20
    for p in (0.1, 0.5, 0.9):
        keep = oracle.dropout_mask(n, p, seed=1234)
        rate = keep.float().mean().item()
        sigma = math.sqrt(p * (1 - p) / n)
        assert abs(rate - (1 - p)) < 5 * sigma + 2.0**-16, (p, rate)
        # every one of the eight 16-bit lanes of a Philox call has that rate
        lanes = keep.view(-1, 8).float().mean(0)
        assert (lanes - (1 - p)).abs().max().item() < 5 * sigma * math.sqrt(8) + 2.0**-16
        # neighbours are uncorrelated
        k = keep.float() - (1 - p)
        assert abs((k[:-1] * k[1:]).mean().item()) < 5 * p * (1 - p) / math.sqrt(n)
    base = oracle.dropout_mask(4096, 0.5, seed=1)
    assert not torch.equal(base, oracle.dropout_mask(4096, 0.5, seed=2))
    assert not torch.equal(base, oracle.dropout_mask(4096, 0.5, seed=1, offset=1))
    assert not torch.equal(base, oracle.dropout_mask(4096, 0.5, seed=1 << 32))
    assert torch.equal(base, oracle.dropout_mask(4096, 0.5, seed=1))
    assert torch.equal(base[:1000], oracle.dropout_mask(1000, 0.5, seed=1))          # a prefix, whatever the length
    assert oracle.dropout_mask(4096, 0.0, seed=7).all()
    # the mask is monotone in p: what is dropped at p stays dropped at p' > p
    assert not (oracle.dropout_mask(4096, 0.7, seed=1) & ~oracle.dropout_mask(4096, 0.3, seed=1)).any()


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_dropout_add_with_dropout(dtype):
    x, bias = inputs(dtype, rows=33, cols=40, seed=21)
    res = util.randn(x.shape, dtype, seed=22, std=2.0)
    p, seed = 0.25, 99
    keep = oracle.dropout_mask(x.numel(), p, seed).view_as(x)
    out = oracle.bias_dropout_add(x, bias, res, p, seed)
    # torch's definition of dropout applied with this mask, in fp32
    scale = torch.tensor(1.0 / (1.0 - p), dtype=torch.float64).float()
    want = (res.float() + torch.where(keep, (x.float() + bias.float()) * scale, torch.zeros(()))).to(dtype)
    assert torch.equal(util.raw_bits(out), util.raw_bits(want))
    assert torch.equal(util.raw_bits(out)[~keep], util.raw_bits(res)[~keep])
    # p = 0 is the deterministic function; without bias and residual it is the backward of the dropout
    assert torch.equal(util.raw_bits(oracle.bias_dropout_add(x, bias, res, 0.0, seed)),
                       util.raw_bits(oracle.bias_add_residual(x, bias, res)))
    g = oracle.bias_dropout_add(x, None, None, p, seed)
    assert torch.equal(util.raw_bits(g), util.raw_bits(torch.where(keep, x.float() * scale, torch.zeros(())).to(dtype)))
    # the expectation is preserved: mean over many seeds of dropout(v) approaches v
    v = torch.ones((1, 64), dtype=torch.float32)
    mean = sum(oracle.bias_dropout_add(v, None, None, 0.5, s) for s in range(400)) / 400
    assert (mean - 1).abs().max().item() < 0.5
    assert abs(mean.mean().item() - 1) < 0.05


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_add_residual_pair_is_three_fused_calls(dtype):
    """residual + ((x1 + b1) + (x2 + b2)) rounded where the parallel-residual layer's three bias_dropout_add calls
    round when each runs as one fused function (fp32 inside, one rounding at its end; dropout off):
    megatron/model/transformer.py:1229-1250, fused_bias_dropout.py:28-60. Written out with torch in fp32."""
    rows, cols = 37, 48
    x1, x2, res = (util.randn((rows, cols), dtype, seed=60 + i, std=2.0) for i in range(3))
    b1, b2 = (util.randn((cols,), dtype, seed=70 + i) for i in range(2))

    def call(x, bias, residual):      # one bias_dropout_add: fp32 inside, rounded once
        v = x.float() if bias is None else x.float() + bias.float()
        return (v if residual is None else residual.float() + v).to(dtype)

    for ba, bb in ((b1, b2), (None, b2), (b1, None), (None, None)):
        t1 = x1 if ba is None else call(x1, ba, None)
        want = call(call(x2, bb, t1), None, res)
        got = oracle.bias_add_residual_pair(x1, ba, x2, bb, res)
        assert torch.equal(util.raw_bits(got), util.raw_bits(want)), (ba is None, bb is None)
    if dtype != torch.float32:   # and the roundings matter: one rounding at the very end gives other bits somewhere
        once = (res.float() + ((x1.float() + b1.float()) + (x2.float() + b2.float()))).to(dtype)
        assert not torch.equal(util.raw_bits(once), util.raw_bits(oracle.bias_add_residual_pair(x1, b1, x2, b2, res)))
