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
