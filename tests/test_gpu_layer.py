"""GPU parity of the element-wise layer kernels (bias + tanh-GeLU forward/backward
with the fused bias gradient, bias + residual add) through the C ABI and the
Python functions, against the CPU oracle.

Tolerances: GeLU results within 2 representable values of the oracle, or within the
fp32 rounding noise the reference's own expression carries (util.gelu_noise);
bias + residual add bit-exact; column sums within fp32 summation noise."""
import ctypes

import pytest
import torch
import torch.nn.functional as F

import oracle
import util

pytestmark = pytest.mark.gpu
DEV = "cuda"
DTYPES = [torch.bfloat16, torch.float16, torch.float32]
IDS = ["bf16", "fp16", "fp32"]


def ptr(t):
    return None if t is None else t.data_ptr()


def abi_gelu_fwd(hp, y, bias, out=None):
    out = torch.empty_like(y) if out is None else out
    cols = y.size(-1)
    rc = hp.lib().nhp_bias_gelu_fwd(out.data_ptr(), y.data_ptr(), ptr(bias), y.numel() // cols, cols,
                                    hp.dtype_code(y, "t"), None)
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return out


def abi_gelu_bwd(hp, g, y, bias, with_dbias=True):
    dx = torch.empty_like(y)
    cols = y.size(-1)
    rows = y.numel() // cols
    code = hp.dtype_code(y, "t")
    dbias = torch.full((cols,), float("nan"), dtype=y.dtype, device=y.device) if with_dbias else None
    nbytes = hp.lib().nhp_bias_gelu_bwd_workspace_bytes(rows, cols, code)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=y.device) if with_dbias else None
    rc = hp.lib().nhp_bias_gelu_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), ptr(bias), ptr(dbias), ptr(ws),
                                    rows, cols, code, None)
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return dx, dbias


# rows, cols: wide and narrow tiles, partial tiles, column counts that are not a multiple of the chunk
SHAPES = [(1, 8), (3, 16), (37, 96), (5, 1000), (300, 2048), (64, 8192), (1000, 24), (129, 2056), (7, 4100), (2, 5)]


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_bias_gelu_forward_backward_vs_oracle(hotpath, shape, dtype):
    rows, cols = shape
    print(f"bias_gelu case {shape} {dtype}", flush=True)
    y = util.randn((rows, cols), dtype, seed=rows + cols, std=3.0)
    bias = util.randn((cols,), dtype, seed=cols, std=0.5)
    g = util.randn((rows, cols), dtype, seed=rows, std=1.0)
    x32 = bias.float() + y.float()
    got = abi_gelu_fwd(hotpath, y.to(DEV), bias.to(DEV)).cpu()
    util.assert_close_ulp_or_noise(got, oracle.bias_gelu_fwd(y, bias), 2, util.gelu_noise(x32), "fwd")
    dx, dbias = abi_gelu_bwd(hotpath, g.to(DEV), y.to(DEV), bias.to(DEV))
    dx, dbias = dx.cpu(), dbias.cpu()
    util.assert_close_ulp_or_noise(dx, oracle.bias_gelu_bwd(g, y, bias), 2, util.gelu_noise(x32, g), "bwd")
    # the bias gradient is the column sum of the dx that was stored
    noise = dx.float().abs().sum(0) * 16 * util.EPS32
    util.assert_close_ulp_or_noise(dbias, oracle.column_sum(dx), 1, noise, "dbias")
    dx_only, none = abi_gelu_bwd(hotpath, g.to(DEV), y.to(DEV), bias.to(DEV), with_dbias=False)
    assert none is None and torch.equal(util.raw_bits(dx_only.cpu()), util.raw_bits(dx))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_bias_gelu_edge_cases(hotpath, dtype):
    # no bias, special values, in place, unaligned pointers, empty tensors
    v = torch.tensor([[0.0, -0.0, 30.0, -30.0, float("inf"), float("-inf"), float("nan"), 1.0]], dtype=dtype)
    got = abi_gelu_fwd(hotpath, v.to(DEV), None).cpu()
    want = oracle.bias_gelu_fwd(v, None)
    util.assert_ulp_close(got, want, 2, "special values")
    # the derivative stays finite (0 on the far left, 1 on the far right) wherever x * x is finite
    big = [0.0, -0.0, 1.0, 30.0, -30.0, 1e4, -1e4] + ([] if dtype == torch.float16 else [1e13, -1e13, 1e15, -1e15, 1e18, -1e18])
    v = torch.tensor([big + [0.5] * (16 - len(big))], dtype=dtype)
    g = torch.full_like(v, 1.5)
    dx, _ = abi_gelu_bwd(hotpath, g.to(DEV), v.to(DEV), None, with_dbias=False)
    want = oracle.bias_gelu_bwd(g, v, None)
    assert torch.isfinite(dx.cpu().float()).all()
    util.assert_ulp_close(dx.cpu(), want, 2, "derivative at large inputs")
    y = util.randn((40, 256), dtype, seed=1, std=3.0)
    yd = y.to(DEV)
    inplace = abi_gelu_fwd(hotpath, yd, None, out=yd).cpu()
    util.assert_close_ulp_or_noise(inplace, oracle.bias_gelu_fwd(y, None), 2, util.gelu_noise(y), "in place")
    # a view that starts one element into a buffer is not 16-byte aligned
    buf = torch.zeros(40 * 256 + 8, dtype=dtype, device=DEV)
    shifted = buf[1:1 + 40 * 256].view(40, 256)
    shifted.copy_(y)
    util.assert_close_ulp_or_noise(abi_gelu_fwd(hotpath, shifted, None).cpu(), oracle.bias_gelu_fwd(y, None), 2,
                                   util.gelu_noise(y), "unaligned")
    empty = torch.empty((0, 64), dtype=dtype, device=DEV)
    assert abi_gelu_fwd(hotpath, empty, None).shape == (0, 64)


def test_bias_gelu_results_are_reproducible(hotpath):
    y = util.randn((777, 2048), torch.bfloat16, seed=1, std=3.0).to(DEV)
    bias = util.randn((2048,), torch.bfloat16, seed=2).to(DEV)
    g = util.randn((777, 2048), torch.bfloat16, seed=3).to(DEV)
    first = abi_gelu_bwd(hotpath, g, y, bias)
    for _ in range(3):
        again = abi_gelu_bwd(hotpath, g, y, bias)
        assert torch.equal(util.raw_bits(first[0]), util.raw_bits(again[0]))
        assert torch.equal(util.raw_bits(first[1]), util.raw_bits(again[1]))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_gelu_function_autograd(dtype):
    """bias_gelu_impl under autograd: output, input gradient and the reduced bias gradient against
    torch's own tanh-GeLU evaluated in fp32 on the same device."""
    from megatron.model.activations import bias_gelu, bias_gelu_back, bias_gelu_impl

    s, b, h = 64, 3, 1024
    y = util.randn((s, b, h), dtype, seed=1, std=2.0).to(DEV).requires_grad_(True)
    bias = util.randn((h,), dtype, seed=2, std=0.5).to(DEV).requires_grad_(True)
    g = util.randn((s, b, h), dtype, seed=3).to(DEV)
    out = bias_gelu_impl(y, bias)
    out.backward(g)
    assert out.shape == (s, b, h) and y.grad.shape == (s, b, h) and bias.grad.shape == (h,)
    yr = y.detach().float().requires_grad_(True)
    br = bias.detach().float().requires_grad_(True)
    ref = F.gelu(yr + br, approximate="tanh")
    ref.backward(g.float())
    x32 = (yr + br).detach().cpu()
    util.assert_close_ulp_or_noise(out.detach().cpu(), ref.detach().to(dtype).cpu(), 2, util.gelu_noise(x32), "out")
    util.assert_close_ulp_or_noise(y.grad.cpu(), yr.grad.to(dtype).cpu(), 2, util.gelu_noise(x32, g.cpu()), "dx")
    # the reduced gradient sums rounded values: compare with the fp32 sum within the rounding of s*b terms
    tol = (yr.grad.abs().sum(dim=(0, 1)) * 2.0 ** (-8 if dtype == torch.bfloat16 else -11)).cpu()
    assert torch.all((bias.grad.float().cpu() - br.grad.cpu()).abs() <= tol + 1e-6)
    # the two plain functions
    assert torch.equal(util.raw_bits(bias_gelu(bias.detach(), y.detach()).cpu()), util.raw_bits(out.detach().cpu()))
    assert torch.equal(util.raw_bits(bias_gelu_back(g, bias.detach(), y.detach()).cpu()), util.raw_bits(y.grad.cpu()))


def test_bias_gelu_rejects_cpu_tensors_and_mismatches():
    from megatron.model.activations import bias_gelu

    with pytest.raises(RuntimeError):
        bias_gelu(torch.zeros(8), torch.zeros(4, 8))
    with pytest.raises(RuntimeError):
        bias_gelu(torch.zeros(4, device=DEV), torch.zeros(4, 8, device=DEV))
    with pytest.raises(RuntimeError):
        bias_gelu(torch.zeros(8, device=DEV, dtype=torch.float16), torch.zeros(4, 8, device=DEV))


def test_bias_gelu_full_size(hotpath):
    """The MLP activation of the 1.4B configuration: [2048*8, 8192] bf16. Sampled rows against the
    oracle, everything against torch's fp32 tanh-GeLU on the device."""
    rows, cols = 2048 * 8, 8192
    gen = torch.Generator(device=DEV).manual_seed(0)
    y = (torch.randn((rows, cols), generator=gen, device=DEV) * 2).bfloat16()
    bias = (torch.randn((cols,), generator=gen, device=DEV) * 0.5).bfloat16()
    g = torch.randn((rows, cols), generator=gen, device=DEV).bfloat16()
    out = abi_gelu_fwd(hotpath, y, bias)
    dx, dbias = abi_gelu_bwd(hotpath, g, y, bias)
    pick = torch.tensor([0, 1, 31, 32, 4095, 9000, rows - 1])
    yc, gc, bc = y[pick.to(DEV)].cpu(), g[pick.to(DEV)].cpu(), bias.cpu()
    x32 = bc.float() + yc.float()
    util.assert_close_ulp_or_noise(out[pick.to(DEV)].cpu(), oracle.bias_gelu_fwd(yc, bc), 2, util.gelu_noise(x32), "fwd")
    util.assert_close_ulp_or_noise(dx[pick.to(DEV)].cpu(), oracle.bias_gelu_bwd(gc, yc, bc), 2,
                                   util.gelu_noise(x32, gc), "bwd")
    ref = F.gelu(y.float() + bias.float(), approximate="tanh")
    err = (out.float() - ref).abs()
    assert bool((err <= 2.0**-7 * ref.abs() + 1e-6).all())
    del ref, err
    want_dbias = dx.float().sum(0)
    scale = dx.float().abs().sum(0)
    assert bool(((dbias.float() - want_dbias).abs() <= 2.0**-8 * want_dbias.abs() + scale * 16 * util.EPS32).all())


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(1, 8), (37, 96), (5, 1000), (300, 2048), (1000, 24), (64, 8192)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_bias_add_residual_bit_exact(hotpath, shape, dtype):
    rows, cols = shape
    x = util.randn((rows, cols), dtype, seed=1, std=2.0)
    bias = util.randn((cols,), dtype, seed=2)
    res = util.randn((rows, cols), dtype, seed=3, std=2.0)
    xd = x.to(DEV)
    for b, r in ((bias, res), (None, res), (bias, None), (None, None)):
        out = torch.empty((rows, cols), dtype=dtype, device=DEV)
        bd = None if b is None else b.to(DEV)  # named, so that the device copies outlive the launch
        rd = None if r is None else r.to(DEV)
        rc = hotpath.lib().nhp_bias_add_residual(out.data_ptr(), xd.data_ptr(), ptr(bd), ptr(rd), rows, cols,
                                                 hotpath.dtype_code(x, "t"), None)
        assert rc == 0
        assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(oracle.bias_add_residual(x, b, r)))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(1, 8), (37, 96), (5, 1000), (300, 2048), (1000, 24), (64, 8192), (3, 1001),
                                   (600000, 8)],   # more row steps than a grid has rows: workgroups loop
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_bias_add_residual_pair_bit_exact(hotpath, shape, dtype):
    """nhp_bias_add_residual_pair against the oracle (three rounded additions) and against three
    nhp_bias_add_residual launches, bit for bit; every combination of missing biases; in place on x1."""
    rows, cols = shape
    x1, x2, res = (util.randn((rows, cols), dtype, seed=10 + i, std=2.0) for i in range(3))
    b1, b2 = (util.randn((cols,), dtype, seed=20 + i) for i in range(2))
    L, code = hotpath.lib(), hotpath.dtype_code(x1, "t")
    d1, d2, dr = x1.to(DEV), x2.to(DEV), res.to(DEV)
    for ba, bb in ((b1, b2), (None, b2), (b1, None), (None, None)):
        da = None if ba is None else ba.to(DEV)
        db = None if bb is None else bb.to(DEV)
        out = torch.empty((rows, cols), dtype=dtype, device=DEV)
        assert L.nhp_bias_add_residual_pair(out.data_ptr(), d1.data_ptr(), ptr(da), d2.data_ptr(), ptr(db), dr.data_ptr(),
                                            rows, cols, code, None) == 0
        assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(oracle.bias_add_residual_pair(x1, ba, x2, bb, res)))
        # the three launches it replaces
        t1, t2, t3, o3 = (torch.empty_like(out) for _ in range(4))
        if da is None:
            t1 = d1
        else:
            assert L.nhp_bias_add_residual(t1.data_ptr(), d1.data_ptr(), ptr(da), None, rows, cols, code, None) == 0
        assert L.nhp_bias_add_residual(t3.data_ptr(), d2.data_ptr(), ptr(db), t1.data_ptr(), rows, cols, code, None) == 0
        assert L.nhp_bias_add_residual(o3.data_ptr(), t3.data_ptr(), None, dr.data_ptr(), rows, cols, code, None) == 0
        assert torch.equal(util.raw_bits(out), util.raw_bits(o3))
    inplace = d1.clone()
    assert L.nhp_bias_add_residual_pair(inplace.data_ptr(), inplace.data_ptr(), ptr(b1.to(DEV)), d2.data_ptr(),
                                        ptr(b2.to(DEV)), dr.data_ptr(), rows, cols, code, None) == 0
    assert torch.equal(util.raw_bits(inplace.cpu()), util.raw_bits(oracle.bias_add_residual_pair(x1, b1, x2, b2, res)))


def test_bias_add_residual_pair_function_and_gradients():
    from megatron.model.fused_bias_dropout import bias_add_residual_pair, bias_dropout_add_fused_inference

    dtype = torch.bfloat16
    x1, x2, res = (util.randn((32, 4, 512), dtype, seed=30 + i, std=2.0).to(DEV).requires_grad_(True) for i in range(3))
    b1, b2 = (util.randn((512,), dtype, seed=40 + i).to(DEV).requires_grad_(True) for i in range(2))
    out = bias_add_residual_pair(x1, b1.expand_as(x1), x2, b2, res)     # one bias expanded as the reference passes it
    g = util.randn((32, 4, 512), dtype, seed=50).to(DEV)
    out.backward(g)
    got = [t.grad.clone() for t in (x1, b1, x2, b2, res)]
    for t in (x1, b1, x2, b2, res):
        t.grad = None
    a = bias_dropout_add_fused_inference(x1, b1.expand_as(x1), None, 0.0)
    o = bias_dropout_add_fused_inference(x2, b2, a, 0.0)
    ref = bias_dropout_add_fused_inference(o, None, res, 0.0)
    assert torch.equal(util.raw_bits(out), util.raw_bits(ref))
    ref.backward(g)
    for mine, theirs in zip(got, (x1, b1, x2, b2, res)):
        assert torch.equal(util.raw_bits(mine), util.raw_bits(theirs.grad))
    with pytest.raises(RuntimeError):
        bias_add_residual_pair(x1, b1, x2[:16], b2, res)
    with pytest.raises(RuntimeError):
        bias_add_residual_pair(x1, b1, x2, b2, None)


def test_bias_dropout_add_functions():
    from megatron.model.fused_bias_dropout import (bias_dropout_add_fused_inference, bias_dropout_add_fused_train,
                                                    get_bias_dropout_add)

    dtype = torch.bfloat16
    x = util.randn((32, 4, 512), dtype, seed=1, std=2.0)
    bias = util.randn((512,), dtype, seed=2)
    res = util.randn((32, 4, 512), dtype, seed=3, std=2.0)
    want = oracle.bias_add_residual(x, bias, res)
    xd = x.to(DEV).requires_grad_(True)
    bd = bias.to(DEV).requires_grad_(True)
    rd = res.to(DEV).requires_grad_(True)
    out = bias_dropout_add_fused_inference(xd, bd, rd, 0.1)
    assert torch.equal(util.raw_bits(out.detach().cpu()), util.raw_bits(want))
    g = util.randn(x.shape, dtype, seed=4).to(DEV)
    out.backward(g)
    assert torch.equal(xd.grad, g) and torch.equal(rd.grad, g)
    assert torch.allclose(bd.grad.float(), g.float().sum(dim=(0, 1)), rtol=2.0**-7, atol=1e-2)
    same = bias_dropout_add_fused_train(x.to(DEV), bias.to(DEV), res.to(DEV), 0.0)
    assert torch.equal(util.raw_bits(same.cpu()), util.raw_bits(want))
    assert torch.equal(util.raw_bits(get_bias_dropout_add(False)(x.to(DEV), bias.to(DEV), res.to(DEV), 0.5).cpu()),
                       util.raw_bits(want))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(1, 8), (37, 96), (5, 1000), (300, 2048), (1000, 24), (64, 8192), (3, 7)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_bias_dropout_add_with_dropout_bit_exact(hotpath, shape, dtype):
    """The mask comes from the library's generator, which the oracle restates: same seed, same bits."""
    rows, cols = shape
    x = util.randn((rows, cols), dtype, seed=1, std=2.0)
    bias = util.randn((cols,), dtype, seed=2)
    res = util.randn((rows, cols), dtype, seed=3, std=2.0)
    L, code = hotpath.lib(), hotpath.dtype_code(x, "t")
    xd, bd, rd = x.to(DEV), bias.to(DEV), res.to(DEV)
    for p, seed, offset in ((0.1, 7, 0), (0.5, (1 << 40) + 3, 5), (0.0, 1, 0)):
        out = torch.empty_like(xd)
        assert L.nhp_bias_dropout_add(out.data_ptr(), xd.data_ptr(), bd.data_ptr(), rd.data_ptr(), rows, cols, p, seed, offset,
                                      code, None) == 0
        want = oracle.bias_dropout_add(x, bias, res, p, seed, offset)
        assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(want)), (p, seed)
        dx = torch.empty_like(xd)
        assert L.nhp_dropout_bwd(dx.data_ptr(), xd.data_ptr(), rows, cols, p, seed, offset, code, None) == 0
        assert torch.equal(util.raw_bits(dx.cpu()), util.raw_bits(oracle.bias_dropout_add(x, None, None, p, seed, offset)))
    assert L.nhp_bias_dropout_add(out.data_ptr(), xd.data_ptr(), None, None, rows, cols, 1.0, 1, 0, code, None) == -2
    assert L.nhp_bias_dropout_add(out.data_ptr(), xd.data_ptr(), None, None, rows, cols, -0.1, 1, 0, code, None) == -2


def test_bias_dropout_add_training_functions():
    from megatron.model.fused_bias_dropout import bias_dropout_add_fused_train, get_bias_dropout_add

    dtype, p = torch.bfloat16, 0.2
    x = util.randn((64, 4, 1024), dtype, seed=1, std=2.0).to(DEV).requires_grad_(True)
    bias = util.randn((1024,), dtype, seed=2).to(DEV).requires_grad_(True)
    res = util.randn((64, 4, 1024), dtype, seed=3, std=2.0).to(DEV).requires_grad_(True)
    from megatron.model import dropout_rng

    torch.manual_seed(5)
    seed = dropout_rng.next_seed()  # what the module will draw
    torch.manual_seed(5)
    out = bias_dropout_add_fused_train(x, bias, res, p)
    dropped = ~oracle.dropout_mask(x.numel(), p, seed).view(x.shape).to(DEV)
    rate = dropped.float().mean().item()
    assert abs(rate - p) < 0.01
    assert torch.equal(out.detach()[dropped], res.detach()[dropped])
    full = (res.detach().float() + (x.detach().float() + bias.detach().float()) / (1 - p)).to(dtype)
    assert torch.equal(out.detach()[~dropped], full[~dropped])
    g = util.randn(x.shape, dtype, seed=4).to(DEV)
    out.backward(g)
    assert torch.equal(res.grad, g)
    assert (x.grad[dropped] == 0).all()
    assert torch.equal(x.grad[~dropped], (g.float() / (1 - p)).to(dtype)[~dropped])
    assert torch.allclose(bias.grad.float(), x.grad.float().sum(dim=(0, 1)), rtol=2.0**-7, atol=1e-2)
    # repeatable under torch.manual_seed, different from call to call otherwise
    torch.manual_seed(5)
    again = bias_dropout_add_fused_train(x.detach(), bias.detach(), res.detach(), p)
    other = bias_dropout_add_fused_train(x.detach(), bias.detach(), res.detach(), p)
    assert torch.equal(again, out.detach()) and not torch.equal(other, again)
    evaluated = get_bias_dropout_add(False)(x.detach(), bias.detach(), res.detach(), p)
    assert torch.equal(util.raw_bits(evaluated.cpu()),
                       util.raw_bits(oracle.bias_add_residual(x.detach().cpu(), bias.detach().cpu(), res.detach().cpu())))
    with pytest.raises(ValueError):
        bias_dropout_add_fused_train(x.detach(), bias.detach(), res.detach(), 1.0)


# ---------------------------------------------------------------------------
# gated activations
# ---------------------------------------------------------------------------
GATES = ["swiglu", "geglu", "reglu", "glu", "bilinear"]


def abi_gated(hp, inp, dy, bias, act):
    rows, f2 = inp.shape
    f = f2 // 2
    code = hp.dtype_code(inp, "t")
    out = torch.empty((rows, f), dtype=inp.dtype, device=inp.device)
    din = torch.empty_like(inp)
    L = hp.lib()
    rc = L.nhp_gated_act_fwd(out.data_ptr(), inp.data_ptr(), ptr(bias), rows, f, oracle.GATE_ACTS[act], code, None)
    assert rc == 0, L.nhp_status_string(rc)
    rc = L.nhp_gated_act_bwd(din.data_ptr(), dy.data_ptr(), inp.data_ptr(), ptr(bias), rows, f, oracle.GATE_ACTS[act], code, None)
    assert rc == 0, L.nhp_status_string(rc)
    return out, din


@pytest.mark.parametrize("act", GATES)
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(1, 8), (37, 96), (5, 1000), (300, 2048), (19, 5504), (1000, 24), (2, 5)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_gated_activation_vs_oracle(hotpath, shape, dtype, act):
    rows, f = shape
    print(f"gated case {shape} {dtype} {act}", flush=True)
    inp = util.randn((rows, 2 * f), dtype, seed=rows + f, std=2.5)
    dy = util.randn((rows, f), dtype, seed=rows)
    bias = util.randn((2 * f,), dtype, seed=f, std=0.5)
    for b in (None, bias):
        out, din = abi_gated(hotpath, inp.to(DEV), dy.to(DEV), None if b is None else b.to(DEV), act)
        want = oracle.gated_act_fwd(inp, act, b)
        util.assert_close_ulp_or_noise(out.cpu(), want, 2, util.gated_noise(inp, b, act, want), "fwd")
        want_d = oracle.gated_act_bwd(dy, inp, act, b)
        util.assert_close_ulp_or_noise(din.cpu(), want_d, 2, util.gated_noise(inp, b, act, want_d, dy), "bwd")


@pytest.mark.parametrize("act", ["swiglu", "geglu"])
def test_gated_activation_module_autograd(act):
    """Gated_Activation under autograd against the reference's expression in fp32 on the device."""
    import types

    from megatron.model.activations import Gated_Activation, get_activation

    func, gated = get_activation(types.SimpleNamespace(activation=act))
    assert gated
    m = Gated_Activation(func, use_swiglu=(act == "swiglu"))
    dtype, s, b, f = torch.bfloat16, 48, 2, 1376
    x = util.randn((s, b, 2 * f), dtype, seed=1, std=2.0).to(DEV).requires_grad_(True)
    bias = util.randn((2 * f,), dtype, seed=2, std=0.5).to(DEV).requires_grad_(True)
    g = util.randn((s, b, f), dtype, seed=3).to(DEV)
    out = m(x, bias)
    out.backward(g)
    xr = x.detach().float().requires_grad_(True)
    br = bias.detach().float().requires_grad_(True)
    xx, gate = xr.chunk(2, dim=-1)
    b1, b2 = br.chunk(2, dim=-1)
    ref = func(gate + b2) * (xx + b1)
    ref.backward(g.float())
    assert out.shape == (s, b, f) and x.grad.shape == x.shape and bias.grad.shape == bias.shape
    lim = 2.0**-7
    assert (out.float() - ref).norm() <= lim * ref.norm()
    assert (x.grad.float() - xr.grad).norm() <= lim * xr.grad.norm()
    assert (bias.grad.float() - br.grad).norm() <= 2 * lim * br.grad.norm()
    plain = m(x.detach())
    util.assert_close_ulp_or_noise(plain.cpu(), oracle.gated_act_fwd(x.detach().cpu(), act), 2,
                                   util.gated_noise(x.detach().cpu(), None, act, plain.cpu()), "no bias")
    with pytest.raises(ValueError):
        Gated_Activation(torch.tanh)


def test_element_offsets_beyond_32_bits(hotpath):
    """[65544, 65536] bf16 holds more than 2^32 elements: rows near the end must come out like rows near
    the start for bias+GeLU (in place), SwiGLU and LayerNorm."""
    rows, cols = 65544, 65536
    L, BF16 = hotpath.lib(), hotpath.BF16
    gen = torch.Generator(device=DEV).manual_seed(0)
    block = (torch.randn((8, cols), generator=gen, device=DEV) * 2).bfloat16()
    x = torch.empty((rows, cols), dtype=torch.bfloat16, device=DEV)
    x.view(-1, 8, cols)[:] = block                       # every group of 8 rows holds the same data
    bias = (torch.randn((cols,), generator=gen, device=DEV) * 0.5).bfloat16()
    want = oracle.bias_gelu_fwd(block.cpu(), bias.cpu())
    noise = util.gelu_noise(bias.float().cpu() + block.float().cpu())
    # SwiGLU first (x is still intact): [rows, 2 * 32768] -> [rows, 32768]
    sw = torch.empty((rows, cols // 2), dtype=torch.bfloat16, device=DEV)
    assert L.nhp_gated_act_fwd(sw.data_ptr(), x.data_ptr(), None, rows, cols // 2, 0, BF16, None) == 0
    want_sw = oracle.gated_act_fwd(block.cpu(), "swiglu")
    for r0 in (0, rows - 8):
        util.assert_close_ulp_or_noise(sw[r0:r0 + 8].cpu(), want_sw, 2, util.gated_noise(block.cpu(), None, "swiglu", want_sw),
                                       f"swiglu rows {r0}")
    del sw
    # LayerNorm into a second tensor
    y = torch.empty_like(x)
    assert L.nhp_layernorm_fwd(y.data_ptr(), None, None, x.data_ptr(), None, None, 1e-5, rows, cols, BF16, BF16, None) == 0
    want_ln, _, _ = oracle.layernorm_fwd(block.cpu(), None, None, 1e-5)
    for r0 in (0, 32768, rows - 8):
        util.assert_close_ulp_or_noise(y[r0:r0 + 8].cpu(), want_ln, 2, torch.full((8, cols), 64 * util.EPS32), f"layernorm rows {r0}")
    del y
    # bias + GeLU in place
    assert L.nhp_bias_gelu_fwd(x.data_ptr(), x.data_ptr(), bias.data_ptr(), rows, cols, BF16, None) == 0
    for r0 in (0, 32768, rows - 8):
        util.assert_close_ulp_or_noise(x[r0:r0 + 8].cpu(), want, 2, noise, f"gelu rows {r0}")
    assert torch.equal(x[:8], x[rows - 8:])


def test_python_functions_accept_non_contiguous_inputs():
    """The Python functions make their inputs contiguous themselves (the reference's TorchScript functions take
    any strides): a transposed view gives the same bits as its contiguous copy."""
    from megatron.model.activations import Gated_Activation, bias_gelu_impl
    from megatron.model.fused_bias_dropout import bias_dropout_add_fused_inference
    from megatron.model.norms import LayerNorm, RMSNorm

    dtype = torch.bfloat16
    base = util.randn((6, 40, 512), dtype, seed=1, std=2.0).to(DEV)
    view = base.transpose(0, 1)                      # [40, 6, 512], not contiguous
    assert not view.is_contiguous()
    bias = util.randn((512,), dtype, seed=2).to(DEV)
    res = util.randn((40, 6, 512), dtype, seed=3).to(DEV)
    ln = LayerNorm(512).to(DEV).to(dtype)
    rms = RMSNorm(512).to(DEV)
    gate = Gated_Activation("swiglu")
    for fn in (lambda t: bias_gelu_impl(t, bias), lambda t: bias_dropout_add_fused_inference(t, bias, res, 0.0), ln, rms,
               lambda t: gate(t, bias)):
        a, b = fn(view), fn(view.contiguous())
        assert a.shape == b.shape and a.shape[:2] == (40, 6)
        assert torch.equal(util.raw_bits(a), util.raw_bits(b))
    # and gradients flow back to a non-contiguous leaf
    leaf = base.clone().requires_grad_(True)
    ln(leaf.transpose(0, 1)).sum().backward()
    assert leaf.grad.shape == leaf.shape and torch.isfinite(leaf.grad.float()).all()


@pytest.mark.parametrize("prob", [0.0, 0.3], ids=["no-dropout", "dropout"])
def test_bias_dropout_add_takes_the_expanded_bias_of_the_reference_call_sites(prob):
    """The reference's layer passes ``bias.expand_as(residual)`` (megatron/model/transformer.py:1229, 1271): same
    result as the vector, and the gradient reaches the vector through autograd's sum over the expansion."""
    from megatron.model.fused_bias_dropout import bias_dropout_add_fused_train

    dtype = torch.bfloat16
    x = util.randn((24, 3, 256), dtype, seed=1).to(DEV).requires_grad_(True)
    res = util.randn((24, 3, 256), dtype, seed=2).to(DEV).requires_grad_(True)
    g = util.randn((24, 3, 256), dtype, seed=3).to(DEV)
    va = util.randn((256,), dtype, seed=4).to(DEV).requires_grad_(True)
    vb = va.detach().clone().requires_grad_(True)
    torch.manual_seed(11)
    a = bias_dropout_add_fused_train(x, va.expand_as(res), res, prob)
    a.backward(g)
    ga, gx, gr = va.grad.clone(), x.grad.clone(), res.grad.clone()
    x.grad = res.grad = None
    torch.manual_seed(11)
    b = bias_dropout_add_fused_train(x, vb, res, prob)
    b.backward(g)
    assert torch.equal(a, b) and torch.equal(gx, x.grad) and torch.equal(gr, res.grad)
    assert ga.shape == (256,)
    # both are sums of the same 72 bf16 values per column, formed in different orders and widths
    assert torch.allclose(ga.float(), vb.grad.float(), rtol=2.0 ** -6, atol=2.0 ** -6)
    with pytest.raises(RuntimeError, match="one value per feature"):
        bias_dropout_add_fused_train(x, torch.zeros_like(res), res, prob)   # a genuinely full-size "bias"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(1, 8), (37, 64), (1000, 512), (4097, 2048), (16, 8192), (33, 1000), (5, 20)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_column_sum_vs_oracle(hotpath, shape, dtype):
    """nhp_column_sum: fp32 accumulation, one rounding; against the oracle's pairwise sum, within the fp32
    noise of a sum of `rows` terms formed in another order. Reproducible from run to run."""
    rows, cols = shape
    print(f"column sum {shape} {dtype}", flush=True)
    x = util.randn((rows, cols), dtype, seed=rows + cols, std=2.0)
    xd = x.to(DEV)
    L, code = hotpath.lib(), hotpath.dtype_code(xd, "t")
    ws = torch.empty(max(L.nhp_column_sum_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device=DEV)
    out = torch.full((cols,), float("nan"), dtype=dtype, device=DEV)
    assert L.nhp_column_sum(out.data_ptr(), xd.data_ptr(), ws.data_ptr(), rows, cols, code, None) == 0
    want = oracle.column_sum(x)
    util.assert_close_ulp_or_noise(out.cpu(), want, 1, x.float().abs().sum(0) * 16 * util.EPS32, "column sums")
    again = torch.empty_like(out)
    assert L.nhp_column_sum(again.data_ptr(), xd.data_ptr(), ws.data_ptr(), rows, cols, code, None) == 0
    assert torch.equal(util.raw_bits(out), util.raw_bits(again))


def test_dropout_seeds_follow_the_cuda_generator():
    """dropout_rng.next_seed: restarted by torch.manual_seed, saved and restored with the CUDA generator state,
    advancing only that generator (torch's CPU stream, hence data order, is untouched), no two alike."""
    from megatron.model import dropout_rng as rng

    torch.manual_seed(11)
    cpu_before = torch.get_rng_state().clone()
    a = [rng.next_seed() for _ in range(3)]
    assert torch.equal(torch.get_rng_state(), cpu_before)
    assert len(set(a)) == 3 and all(0 <= v < 2**63 for v in a)
    torch.manual_seed(11)
    assert [rng.next_seed(torch.device(DEV, 0)) for _ in range(3)] == a
    torch.manual_seed(12)
    assert rng.next_seed() not in a
    state = torch.cuda.get_rng_state()
    b = rng.next_seed()
    torch.cuda.set_rng_state(state)
    assert rng.next_seed() == b
    # torch's own device random numbers and the seeds share one stream: neither repeats the other
    torch.manual_seed(11)
    torch.rand(4, device=DEV)
    assert rng.next_seed() != a[0]
