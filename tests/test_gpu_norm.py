"""GPU parity of LayerNorm and RMSNorm (forward, backward with parameter gradients)
through the C ABI and the modules, against the CPU oracle.

Tolerances: outputs and dx within 2 representable values of the oracle, or within a few
fp32 roundings of the terms that are added up (the sums over a row are formed in a
different order); parameter gradients within the fp32 noise of a sum over all rows."""
import types

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


def make(dtype, rows, cols, seed, pdtype):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn((rows, cols), generator=g) * 2 + 0.5).to(dtype)
    dy = torch.randn((rows, cols), generator=g).to(dtype)
    gamma = (1 + 0.3 * torch.randn(cols, generator=g)).to(pdtype)
    beta = (0.2 * torch.randn(cols, generator=g)).to(pdtype)
    return x, dy, gamma, beta


def abi_layernorm(hp, x, dy, gamma, beta, eps, want_params=True):
    rows, cols = x.shape
    code, pcode = hp.dtype_code(x, "t"), hp._DTYPE[(gamma if gamma is not None else x).dtype]
    y = torch.empty_like(x)
    mean = torch.empty(rows, dtype=torch.float32, device=x.device)
    rstd = torch.empty_like(mean)
    L = hp.lib()
    rc = L.nhp_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), ptr(gamma), ptr(beta), eps,
                             rows, cols, code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    dx = torch.empty_like(x)
    pd = gamma.dtype if gamma is not None else x.dtype
    dg = torch.full((cols,), float("nan"), dtype=pd, device=x.device) if want_params else None
    db = torch.full((cols,), float("nan"), dtype=pd, device=x.device) if want_params else None
    ws = torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, code), 1), dtype=torch.uint8, device=x.device)
    rc = L.nhp_layernorm_bwd(dx.data_ptr(), ptr(dg), ptr(db), dy.data_ptr(), x.data_ptr(), mean.data_ptr(),
                             rstd.data_ptr(), ptr(gamma), ws.data_ptr(), rows, cols, code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    return y, mean, rstd, dx, dg, db


def abi_rmsnorm(hp, x, dy, scale, offset, eps, mode, stat=None, want_params=True):
    if stat is not None:
        return abi_rmsnorm_partial(hp, x, dy, scale, offset, eps, mode, stat)
    rows, cols = x.shape
    code, pcode = hp.dtype_code(x, "t"), hp._DTYPE[(scale if scale is not None else x).dtype]
    y = torch.empty_like(x)
    inv = torch.empty(rows, dtype=torch.float32, device=x.device)
    L = hp.lib()
    rc = L.nhp_rmsnorm_fwd(y.data_ptr(), inv.data_ptr(), x.data_ptr(), ptr(scale), ptr(offset), eps, mode, rows, cols,
                           code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    dx = torch.empty_like(x)
    pd = scale.dtype if scale is not None else x.dtype
    ds = torch.full((cols,), float("nan"), dtype=pd, device=x.device) if want_params else None
    do = torch.full((cols,), float("nan"), dtype=pd, device=x.device) if want_params else None
    ws = torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, code), 1), dtype=torch.uint8, device=x.device)
    rc = L.nhp_rmsnorm_bwd(dx.data_ptr(), ptr(ds), ptr(do), dy.data_ptr(), x.data_ptr(), inv.data_ptr(),
                           ptr(scale), ws.data_ptr(), eps, mode, rows, cols, code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    return y, inv, dx, ds, do


def abi_rmsnorm_partial(hp, x, dy, scale, offset, eps, mode, stat):
    rows, cols = x.shape
    code, pcode = hp.dtype_code(x, "t"), hp._DTYPE[(scale if scale is not None else x).dtype]
    y = torch.empty_like(x)
    inv = torch.empty(rows, dtype=torch.float32, device=x.device)
    L = hp.lib()
    rc = L.nhp_rmsnorm_partial_fwd(y.data_ptr(), inv.data_ptr(), x.data_ptr(), ptr(scale), ptr(offset), eps, mode, rows,
                                   cols, stat, code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    dx = torch.empty_like(x)
    pd = scale.dtype if scale is not None else x.dtype
    ds = torch.full((cols,), float("nan"), dtype=pd, device=x.device)
    do = torch.full((cols,), float("nan"), dtype=pd, device=x.device)
    ws = torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, code), 1), dtype=torch.uint8, device=x.device)
    rc = L.nhp_rmsnorm_partial_bwd(dx.data_ptr(), ds.data_ptr(), do.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                   inv.data_ptr(), ptr(scale), ws.data_ptr(), eps, mode, rows, cols, stat, code, pcode,
                                   None)
    assert rc == 0, L.nhp_status_string(rc)
    return y, inv, dx, ds, do


def out_noise(gamma, like):
    g = gamma.float().abs() if gamma is not None else torch.ones(like.size(-1))
    return (g * 64 * util.EPS32).expand_as(like.float())


def dx_noise(dy, gamma, factor):
    g = gamma.float().abs() if gamma is not None else 1.0
    return ((dy.float().abs() * g).sum(-1, keepdim=True) * factor[:, None] * 64 * util.EPS32).expand_as(dy.float())


# rows, cols: every geometry (lanes per row 1..64, 1..16 waves per row), partial row blocks, scalar fallbacks
SHAPES = [(5, 8), (9, 16), (33, 64), (70, 128), (300, 512), (37, 1024), (129, 2048), (21, 4096), (19, 8192),
          (7, 16384), (3, 32768), (11, 1000), (4, 65536), (13, 2056), (1, 24),
          # hidden sizes that are not a power of two: workgroups of 3, 5 and 6 waves per row
          (23, 2560), (17, 3072), (13, 5120), (11, 6144), (9, 1536)]


@pytest.mark.parametrize("pd", ["same", "fp32"])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_layernorm_vs_oracle(hotpath, shape, dtype, pd):
    rows, cols = shape
    if pd == "fp32" and dtype == torch.float32:
        pytest.skip("same case")
    pdtype = dtype if pd == "same" else torch.float32
    print(f"layernorm case {shape} {dtype} params {pdtype}", flush=True)
    x, dy, gamma, beta = make(dtype, rows, cols, rows + cols, pdtype)
    eps = 1e-5
    want_y, want_mean, want_rstd = oracle.layernorm_fwd(x, gamma, beta, eps)
    y, mean, rstd, dx, dg, db = [t.cpu() for t in abi_layernorm(hotpath, x.to(DEV), dy.to(DEV), gamma.to(DEV),
                                                                  beta.to(DEV), eps)]
    util.assert_close_ulp_or_noise(y, want_y, 2, out_noise(gamma, x), "y")
    assert torch.allclose(mean, want_mean, rtol=0, atol=2e-6 * (1 + x.float().abs().max().item()))
    assert torch.allclose(rstd, want_rstd, rtol=1e-5, atol=0)
    # backward from the statistics the GPU produced, against the oracle fed with the same statistics
    want_dx, want_dg, want_db = oracle.layernorm_bwd(dy, x, mean, rstd, gamma)
    util.assert_close_ulp_or_noise(dx, want_dx, 2, dx_noise(dy, gamma, rstd), "dx")
    col = (dy.float().abs() * ((x.float() - mean[:, None]) * rstd[:, None]).abs()).sum(0) * 32 * util.EPS32
    util.assert_close_ulp_or_noise(dg, want_dg, 2, col, "dgamma")
    util.assert_close_ulp_or_noise(db, want_db, 2, dy.float().abs().sum(0) * 32 * util.EPS32, "dbeta")
    # without parameter gradients another instantiation runs (smaller workgroups, no column sums): the same dx bit for bit
    alone = abi_layernorm(hotpath, x.to(DEV), dy.to(DEV), gamma.to(DEV), beta.to(DEV), eps, want_params=False)[3].cpu()
    assert torch.equal(util.raw_bits(alone), util.raw_bits(dx)), "dx without parameter gradients"


def abi_layernorm_pair(hp, x, dy1, dy2, gamma1, beta1, gamma2, beta2, eps, want=(True, True, True, True)):
    rows, cols = x.shape
    code, pcode = hp.dtype_code(x, "t"), hp._DTYPE[gamma1.dtype]
    y1, y2 = torch.empty_like(x), torch.empty_like(x)
    mean = torch.empty(rows, dtype=torch.float32, device=x.device)
    rstd = torch.empty_like(mean)
    L = hp.lib()
    rc = L.nhp_layernorm_pair_fwd(y1.data_ptr(), y2.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), ptr(gamma1),
                                  ptr(beta1), ptr(gamma2), ptr(beta2), eps, rows, cols, code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    dx = torch.empty_like(x)
    grads = [torch.full((cols,), float("nan"), dtype=gamma1.dtype, device=x.device) if w else None for w in want]
    ws = torch.empty(max(L.nhp_layernorm_pair_bwd_workspace_bytes(rows, cols, code), 1), dtype=torch.uint8, device=x.device)
    rc = L.nhp_layernorm_pair_bwd(dx.data_ptr(), ptr(grads[0]), ptr(grads[1]), ptr(grads[2]), ptr(grads[3]), dy1.data_ptr(),
                                  dy2.data_ptr(), x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), ptr(gamma1), ptr(gamma2),
                                  ws.data_ptr(), rows, cols, code, pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    return y1, y2, mean, rstd, dx, grads


@pytest.mark.parametrize("pd", ["same", "fp32"])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
def test_layernorm_pair_vs_oracle(hotpath, shape, dtype, pd):
    rows, cols = shape
    if pd == "fp32" and dtype == torch.float32:
        pytest.skip("same case")
    pdtype = dtype if pd == "same" else torch.float32
    print(f"layernorm pair case {shape} {dtype} params {pdtype}", flush=True)
    x, dy1, gamma1, beta1 = make(dtype, rows, cols, rows + cols, pdtype)
    _, dy2, gamma2, beta2 = make(dtype, rows, cols, rows + cols + 1, pdtype)
    eps = 1e-5
    dev = [t.to(DEV) for t in (x, dy1, dy2, gamma1, beta1, gamma2, beta2)]
    y1, y2, mean, rstd, dx, grads = abi_layernorm_pair(hotpath, *dev, eps)
    # the statistics and outputs of two single launches (whose sums over a row may be formed in another order)
    s1 = abi_layernorm(hotpath, dev[0], dev[1], dev[3], dev[4], eps)
    s2 = abi_layernorm(hotpath, dev[0], dev[2], dev[5], dev[6], eps)
    util.assert_close_ulp_or_noise(y1.cpu(), s1[0].cpu(), 1, out_noise(gamma1, x), "y1 vs single")
    util.assert_close_ulp_or_noise(y2.cpu(), s2[0].cpu(), 1, out_noise(gamma2, x), "y2 vs single")
    assert torch.allclose(mean, s1[1], rtol=0, atol=2e-6 * (1 + x.float().abs().max().item()))
    assert torch.allclose(rstd, s1[2], rtol=1e-5, atol=0)
    want_y1, want_y2, _, _ = oracle.layernorm_pair_fwd(x, gamma1, beta1, gamma2, beta2, eps)
    util.assert_close_ulp_or_noise(y1.cpu(), want_y1, 2, out_noise(gamma1, x), "y1")
    util.assert_close_ulp_or_noise(y2.cpu(), want_y2, 2, out_noise(gamma2, x), "y2")
    mean, rstd = mean.cpu(), rstd.cpu()
    want = oracle.layernorm_pair_bwd(dy1, dy2, x, mean, rstd, gamma1, gamma2)
    noise = dx_noise(dy1, gamma1, rstd) + dx_noise(dy2, gamma2, rstd)
    util.assert_close_ulp_or_noise(dx.cpu(), want[0], 2, noise, "dx")
    xhat = ((x.float() - mean[:, None]) * rstd[:, None]).abs()
    for i, dy in ((0, dy1), (2, dy2)):
        util.assert_close_ulp_or_noise(grads[i].cpu(), want[1 + i], 2, (dy.float().abs() * xhat).sum(0) * 32 * util.EPS32,
                                       f"dgamma{i // 2 + 1}")
        util.assert_close_ulp_or_noise(grads[i + 1].cpu(), want[2 + i], 2, dy.float().abs().sum(0) * 32 * util.EPS32,
                                       f"dbeta{i // 2 + 1}")
    # and a second run reproduces every result (fixed summation order)
    again = abi_layernorm_pair(hotpath, *dev, eps)
    assert torch.equal(again[4], dx) and all(torch.equal(a, b) for a, b in zip(again[5], grads))
    # without any parameter gradient (another instantiation: smaller workgroups, no column sums) the same dx bit for bit
    alone = abi_layernorm_pair(hotpath, *dev, eps, want=(False, False, False, False))
    assert torch.equal(util.raw_bits(alone[4]), util.raw_bits(dx)), "dx without parameter gradients"


def test_layernorm_pair_optional_gradients_and_module(hotpath):
    from megatron.model.norms import LayerNorm, layer_norm_pair
    x, dy1, gamma1, beta1 = [t.to(DEV) for t in make(torch.bfloat16, 67, 2048, 5, torch.float32)]
    _, dy2, gamma2, beta2 = [t.to(DEV) for t in make(torch.bfloat16, 67, 2048, 6, torch.float32)]
    full = abi_layernorm_pair(hotpath, x, dy1, dy2, gamma1, beta1, gamma2, beta2, 1e-5)
    for want in ((False, False, False, False), (True, False, False, True), (False, True, True, False)):
        part = abi_layernorm_pair(hotpath, x, dy1, dy2, gamma1, beta1, gamma2, beta2, 1e-5, want=want)
        assert torch.equal(part[4], full[4])
        for got, ref, w in zip(part[5], full[5], want):
            assert (got is None) if not w else torch.equal(got, ref)
    # the module-level helper against two separate modules, gradients through autograd
    torch.manual_seed(3)
    a, b = LayerNorm(2048, eps=1e-5).to(DEV), LayerNorm(2048, eps=1e-5).to(DEV)
    with torch.no_grad():
        a.weight.copy_(gamma1), a.bias.copy_(beta1), b.weight.copy_(gamma2), b.bias.copy_(beta2)
    xa = x.view(1, 67, 2048).clone().requires_grad_(True)
    y1, y2 = layer_norm_pair(xa, a, b)
    (y1 * dy1.view_as(y1)).sum().backward(retain_graph=True)
    only_first = xa.grad.clone()          # the second output unused so far: its gradient arrives as None / zeros
    xa.grad = None
    a.zero_grad(), b.zero_grad()
    ((y1 * dy1.view_as(y1)).sum() + (y2 * dy2.view_as(y2)).sum()).backward()
    pair_grads = [xa.grad.clone(), a.weight.grad.clone(), a.bias.grad.clone(), b.weight.grad.clone(), b.bias.grad.clone()]
    assert torch.equal(pair_grads[0].view(67, 2048), full[4])
    for got, ref in zip(pair_grads[1:], full[5]):
        assert torch.equal(got, ref)
    xb = x.view(1, 67, 2048).clone().requires_grad_(True)
    a.zero_grad(), b.zero_grad()
    z1, z2 = a(xb), b(xb)
    assert util.ulp_distance(z1.cpu(), y1.cpu()).max() <= 1 and util.ulp_distance(z2.cpu(), y2.cpu()).max() <= 1
    (z1 * dy1.view_as(z1)).sum().backward()
    # (kernel-level parity is the test above; here only that the unused second output contributed nothing)
    assert (xb.grad.float() - only_first.float()).abs().max() <= 2 ** -7 * only_first.float().abs().max()
    # different settings fall back to two calls
    c = LayerNorm(2048, eps=1e-6).to(DEV)
    w1, w2 = layer_norm_pair(xb.detach(), a, c)
    assert torch.equal(w1, a(xb.detach())) and torch.equal(w2, c(xb.detach()))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(5, 8), (70, 128), (129, 2048), (21, 4096), (19, 8192), (3, 32768), (11, 1000)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
def test_rmsnorm_vs_oracle(hotpath, shape, dtype, mode):
    rows, cols = shape
    print(f"rmsnorm case {shape} {dtype} mode {mode}", flush=True)
    x, dy, scale, offset = make(dtype, rows, cols, rows + cols + 1, dtype)
    eps = 1e-5 if mode == 0 else 1e-2
    want_y, want_inv = oracle.rmsnorm_fwd(x, scale, offset, eps, mode)
    y, inv, dx, ds, do = [t.cpu() for t in abi_rmsnorm(hotpath, x.to(DEV), dy.to(DEV), scale.to(DEV), offset.to(DEV),
                                                      eps, mode)]
    util.assert_close_ulp_or_noise(y, want_y, 2, out_noise(scale, x), "y")
    assert torch.allclose(inv, want_inv, rtol=1e-5, atol=0)
    want_dx, want_ds, want_do = oracle.rmsnorm_bwd(dy, x, inv, scale, eps, mode)
    util.assert_close_ulp_or_noise(dx, want_dx, 2, dx_noise(dy, scale, inv), "dx")
    col = (dy.float().abs() * (x.float() * inv[:, None]).abs()).sum(0) * 32 * util.EPS32
    util.assert_close_ulp_or_noise(ds, want_ds, 2, col, "dscale")
    util.assert_close_ulp_or_noise(do, want_do, 2, dy.float().abs().sum(0) * 32 * util.EPS32, "doffset")
    alone = abi_rmsnorm(hotpath, x.to(DEV), dy.to(DEV), scale.to(DEV), offset.to(DEV), eps, mode, want_params=False)[2].cpu()
    assert torch.equal(util.raw_bits(alone), util.raw_bits(dx)), "dx without parameter gradients"


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape_stat", [((5, 8), 3), ((70, 128), 32), ((70, 128), 1), ((129, 2048), 512), ((129, 2048), 1023),
                                        ((21, 4096), 4096), ((19, 8192), 2457), ((3, 32768), 16385), ((11, 1000), 333),
                                        ((13, 2056), 2049)],
                         ids=lambda v: f"{v[0][0]}x{v[0][1]}-{v[1]}")
def test_partial_rmsnorm_vs_oracle(hotpath, shape_stat, dtype, mode):
    """Partial RMSNorm: the statistic over the first `stat` columns (chunk-aligned or not, one
    column, all columns), through nhp_rmsnorm_partial_fwd / _bwd."""
    (rows, cols), stat = shape_stat
    print(f"partial rmsnorm case {rows}x{cols} stat {stat} {dtype} mode {mode}", flush=True)
    x, dy, scale, offset = make(dtype, rows, cols, rows + cols + stat, dtype)
    eps = 1e-5 if mode == 0 else 1e-2
    want_y, want_inv = oracle.rmsnorm_fwd(x, scale, offset, eps, mode, stat_cols=stat)
    y, inv, dx, ds, do = [t.cpu() for t in abi_rmsnorm(hotpath, x.to(DEV), dy.to(DEV), scale.to(DEV), offset.to(DEV),
                                                      eps, mode, stat)]
    grow = (x.float().abs() * want_inv[:, None]).clamp(min=1.0)   # columns outside the statistic are not bounded by it
    util.assert_close_ulp_or_noise(y, want_y, 2, out_noise(scale, x) * grow, "y")
    assert torch.allclose(inv, want_inv, rtol=1e-5, atol=0)
    want_dx, want_ds, want_do = oracle.rmsnorm_bwd(dy, x, inv, scale, eps, mode, stat_cols=stat)
    xh = (x.float() * inv[:, None]).abs()
    noise = ((dy.float().abs() * scale.float().abs() * xh).sum(-1, keepdim=True) * xh * inv[:, None] / stat * 256 * util.EPS32
             + dx_noise(dy, scale, inv) / cols)
    util.assert_close_ulp_or_noise(dx, want_dx, 2, noise, "dx")
    col = (dy.float().abs() * xh).sum(0) * 32 * util.EPS32
    util.assert_close_ulp_or_noise(ds, want_ds, 2, col, "dscale")
    util.assert_close_ulp_or_noise(do, want_do, 2, dy.float().abs().sum(0) * 32 * util.EPS32, "doffset")
    if stat == cols:
        full = [t.cpu() for t in abi_rmsnorm(hotpath, x.to(DEV), dy.to(DEV), scale.to(DEV), offset.to(DEV), eps, mode)]
        for a, b in zip((y, inv, dx, ds, do), full):
            assert torch.equal(util.raw_bits(a), util.raw_bits(b))


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("shape", [(9, 16), (70, 128), (129, 2048), (19, 8192), (11, 1000)], ids=lambda s: f"{s[0]}x{s[1]}")
def test_scalenorm_vs_oracle(hotpath, shape, dtype):
    """eps_mode 2: x / max(||x||, eps) * g, with rows whose norm is below eps and an all-zero row."""
    rows, cols = shape
    print(f"scalenorm case {shape} {dtype}", flush=True)
    x, dy, _, _ = make(dtype, rows, cols, rows + cols + 5, dtype)
    x[1] = x[1] * 1e-5          # norm below eps: clamped
    x[2] = 0
    eps = 1e-2
    gvec = torch.full((cols,), 1.7, dtype=dtype)
    want_y, want_inv = oracle.rmsnorm_fwd(x, gvec, None, eps, 2)
    y, inv, dx, ds, _ = [t.cpu() for t in abi_rmsnorm(hotpath, x.to(DEV), dy.to(DEV), gvec.to(DEV), None, eps, 2)]
    util.assert_close_ulp_or_noise(y, want_y, 2, out_noise(gvec, x), "y")
    assert torch.allclose(inv, want_inv, rtol=1e-5, atol=0)
    assert inv[1].item() == pytest.approx(1 / eps) and inv[2].item() == pytest.approx(1 / eps)
    want_dx, want_ds, _ = oracle.rmsnorm_bwd(dy, x, inv, gvec, eps, 2)
    util.assert_close_ulp_or_noise(dx, want_dx, 2, dx_noise(dy, gvec, inv), "dx")
    col = (dy.float().abs() * (x.float() * inv[:, None]).abs()).sum(0) * 32 * util.EPS32
    util.assert_close_ulp_or_noise(ds, want_ds, 2, col, "dscale")


def test_norm_edge_cases(hotpath):
    L = hotpath.lib()
    # no affine terms, no statistics wanted, no parameter gradients, unaligned input, empty tensors
    x, dy, _, _ = make(torch.bfloat16, 50, 256, 3, torch.bfloat16)
    xd, dyd = x.to(DEV), dy.to(DEV)
    y = torch.empty_like(xd)
    rc = L.nhp_layernorm_fwd(y.data_ptr(), None, None, xd.data_ptr(), None, None, 1e-5, 50, 256, 1, 1, None)
    assert rc == 0
    want, mean, rstd = oracle.layernorm_fwd(x, None, None, 1e-5)
    util.assert_close_ulp_or_noise(y.cpu(), want, 2, out_noise(None, x), "plain")
    dx = torch.empty_like(xd)
    mean_d, rstd_d = mean.to(DEV), rstd.to(DEV)  # named, so that the device copies outlive the launch
    rc = L.nhp_layernorm_bwd(dx.data_ptr(), None, None, dyd.data_ptr(), xd.data_ptr(), mean_d.data_ptr(),
                             rstd_d.data_ptr(), None, None, 50, 256, 1, 1, None)
    assert rc == 0
    util.assert_close_ulp_or_noise(dx.cpu(), oracle.layernorm_bwd(dy, x, mean, rstd, None)[0], 2,
                                   dx_noise(dy, None, rstd), "dx without parameters")
    buf = torch.zeros(50 * 256 + 8, dtype=torch.bfloat16, device=DEV)
    shifted = buf[1:1 + 50 * 256].view(50, 256)
    shifted.copy_(xd)
    rc = L.nhp_layernorm_fwd(y.data_ptr(), None, None, shifted.data_ptr(), None, None, 1e-5, 50, 256, 1, 1, None)
    assert rc == 0
    util.assert_close_ulp_or_noise(y.cpu(), want, 2, out_noise(None, x), "unaligned")
    assert L.nhp_layernorm_fwd(None, None, None, None, None, None, 1e-5, 0, 256, 1, 1, None) == 0
    assert L.nhp_layernorm_fwd(y.data_ptr(), None, None, xd.data_ptr(), None, None, 1e-5, 50, 256, 1, 0, None) == -1
    assert L.nhp_rmsnorm_fwd(y.data_ptr(), None, xd.data_ptr(), None, None, 1e-5, 3, 50, 256, 1, 1, None) == -2
    assert L.nhp_rmsnorm_partial_fwd(y.data_ptr(), None, xd.data_ptr(), None, None, 1e-5, 1, 50, 256, 257, 1, 1, None) == -2
    # a constant row (zero variance) and an all-zero row
    const = torch.full((4, 512), 3.0, dtype=torch.bfloat16, device=DEV)
    out = torch.empty_like(const)
    assert L.nhp_layernorm_fwd(out.data_ptr(), None, None, const.data_ptr(), None, None, 1e-5, 4, 512, 1, 1, None) == 0
    assert out.abs().max().item() == 0
    zero = torch.zeros((4, 512), dtype=torch.bfloat16, device=DEV)
    inv = torch.empty(4, dtype=torch.float32, device=DEV)
    for mode in (0, 1):
        assert L.nhp_rmsnorm_fwd(out.data_ptr(), inv.data_ptr(), zero.data_ptr(), None, None, 1e-3, mode, 4, 512, 1, 1, None) == 0
        assert out.abs().max().item() == 0 and torch.isfinite(inv).all()
        ones = torch.ones_like(zero)
        assert L.nhp_rmsnorm_bwd(out.data_ptr(), None, None, ones.data_ptr(), zero.data_ptr(), inv.data_ptr(), None, None,
                                 1e-3, mode, 4, 512, 1, 1, None) == 0
        assert torch.isfinite(out.float()).all()


def test_norm_parameter_gradients_are_reproducible(hotpath):
    x, dy, gamma, beta = [t.to(DEV) for t in make(torch.bfloat16, 5000, 2048, 1, torch.float32)]
    first = abi_layernorm(hotpath, x, dy, gamma, beta, 1e-5)
    for _ in range(3):
        again = abi_layernorm(hotpath, x, dy, gamma, beta, 1e-5)
        for a, b in zip(first, again):
            assert torch.equal(util.raw_bits(a), util.raw_bits(b))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_layernorm_module_matches_torch_module(dtype):
    from megatron.model.norms import LayerNorm

    s, b, h = 96, 4, 2048
    mine = LayerNorm(h, eps=1e-5).to(DEV).to(dtype)
    ref = torch.nn.LayerNorm(h, eps=1e-5).to(DEV).to(dtype)
    with torch.no_grad():
        w = (1 + 0.3 * torch.randn(h, generator=torch.Generator().manual_seed(1))).to(dtype).to(DEV)
        bb = (0.2 * torch.randn(h, generator=torch.Generator().manual_seed(2))).to(dtype).to(DEV)
        for m in (mine, ref):
            m.weight.copy_(w)
            m.bias.copy_(bb)
    x = util.randn((s, b, h), dtype, seed=3, std=2.0).to(DEV)
    g = util.randn((s, b, h), dtype, seed=4).to(DEV)
    xa = x.clone().requires_grad_(True)
    xb = x.clone().requires_grad_(True)
    ya = mine(xa)
    yb = ref(xb)
    ya.backward(g)
    yb.backward(g)
    assert sorted(n for n, _ in mine.named_parameters()) == ["bias", "weight"]
    util.assert_close_ulp_or_noise(ya.detach().cpu(), yb.detach().cpu(), 2, out_noise(w.cpu(), x.cpu()), "y")
    lim = 2.0 ** (-7 if dtype == torch.bfloat16 else -10)
    assert (xa.grad.float() - xb.grad.float()).norm() <= lim * xb.grad.float().norm()
    assert (mine.weight.grad.float() - ref.weight.grad.float()).norm() <= lim * ref.weight.grad.float().norm()
    assert (mine.bias.grad.float() - ref.bias.grad.float()).norm() <= lim * ref.bias.grad.float().norm()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_rmsnorm_module_against_the_reference_expression(dtype):
    """The module against the eager expression of the reference's Python class (autograd through
    torch ops in fp32), and get_norm's choices."""
    from megatron.model.norms import LayerNorm, RMSNorm, get_norm

    s, b, h = 64, 2, 1024
    m = RMSNorm(h, eps=1e-8, bias=True).to(DEV)
    with torch.no_grad():
        m.scale.copy_(1 + 0.3 * torch.randn(h, generator=torch.Generator().manual_seed(1)))
        m.offset.copy_(0.2 * torch.randn(h, generator=torch.Generator().manual_seed(2)))
    assert sorted(n for n, _ in m.named_parameters()) == ["offset", "scale"]
    x = util.randn((s, b, h), dtype, seed=3, std=2.0).to(DEV)
    g = util.randn((s, b, h), dtype, seed=4).to(DEV)
    xa = x.clone().requires_grad_(True)
    y = m(xa)
    y.backward(g)
    xr = x.float().requires_grad_(True)
    sr = m.scale.detach().clone().requires_grad_(True)
    orf = m.offset.detach().clone().requires_grad_(True)
    norm_x = xr.norm(2, dim=-1, keepdim=True)
    rms_x = norm_x * h ** (-1.0 / 2)
    ref = sr * (xr / (rms_x + 1e-8)) + orf
    ref.backward(g.float())
    util.assert_close_ulp_or_noise(y.detach().cpu(), ref.detach().to(dtype).cpu(), 2, out_noise(sr.detach().cpu(), x.cpu()), "y")
    lim = 2.0 ** (-7 if dtype == torch.bfloat16 else -18)
    assert (xa.grad.float() - xr.grad).norm() <= lim * xr.grad.norm()
    assert (m.scale.grad - sr.grad).norm() <= lim * sr.grad.norm()
    assert (m.offset.grad - orf.grad).norm() <= lim * orf.grad.norm()
    args = types.SimpleNamespace(norm="rmsnorm", rms_norm_epsilon=1e-6, rmsnorm_fusion=False, layernorm_epsilon=1e-5)
    cls, eps = get_norm(args)
    assert cls is RMSNorm and eps == 1e-6
    args.norm = "layernorm"
    assert get_norm(args) == (LayerNorm, 1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_partial_rmsnorm_and_scalenorm_modules_against_the_reference_expressions(dtype):
    """RMSNorm(p=0.3) and ScaleNorm against the eager expressions of the reference's classes
    (megatron/model/norms.py:85-107, :117-119) with autograd through torch ops in fp32."""
    from megatron.model.norms import RMSNorm, ScaleNorm

    s, b, h = 64, 2, 1024
    x = util.randn((s, b, h), dtype, seed=3, std=2.0).to(DEV)
    g = util.randn((s, b, h), dtype, seed=4).to(DEV)
    lim = 2.0 ** (-7 if dtype == torch.bfloat16 else -18)

    m = RMSNorm(h, p=0.3, eps=1e-8).to(DEV)
    with torch.no_grad():
        m.scale.copy_(1 + 0.3 * torch.randn(h, generator=torch.Generator().manual_seed(1)))
    part = int(h * 0.3)
    assert m.partial_size == part
    xa = x.clone().requires_grad_(True)
    y = m(xa)
    y.backward(g)
    xr = x.detach().clone().float().requires_grad_(True)
    sr = m.scale.detach().clone().requires_grad_(True)
    partial_x, _ = torch.split(xr, [part, h - part], dim=-1)
    rms_x = partial_x.norm(2, dim=-1, keepdim=True) * part ** (-1.0 / 2)
    ref = sr * (xr / (rms_x + 1e-8))
    ref.backward(g.float())
    grow = (ref.detach().abs() / sr.detach().abs()).clamp(min=1.0).cpu()
    util.assert_close_ulp_or_noise(y.detach().cpu(), ref.detach().to(dtype).cpu(), 2,
                                   out_noise(sr.detach().cpu(), x.cpu()) * grow, "partial y")
    assert (xa.grad.float() - xr.grad).norm() <= lim * xr.grad.norm()
    assert (m.scale.grad - sr.grad).norm() <= lim * sr.grad.norm()

    sn = ScaleNorm(h, eps=1e-5).to(DEV)
    with torch.no_grad():
        sn.g.fill_(1.3)
    xa = x.clone().requires_grad_(True)
    y = sn(xa)
    y.backward(g)
    xr = x.detach().clone().float().requires_grad_(True)
    gr = sn.g.detach().clone().requires_grad_(True)
    n = torch.norm(xr, dim=-1, keepdim=True).clamp(min=1e-5)
    ref = xr / n * gr
    ref.backward(g.float())
    assert y.dtype == dtype and sn.g.grad.shape == (1,)
    util.assert_close_ulp_or_noise(y.detach().cpu(), ref.detach().to(dtype).cpu(), 2,
                                   out_noise(torch.full((h,), 1.3), x.cpu()), "scalenorm y")
    assert (xa.grad.float() - xr.grad).norm() <= lim * xr.grad.norm()
    assert abs(sn.g.grad.item() - gr.grad.item()) <= max(lim, 1e-3) * (g.float() * (xr.detach() / n.detach())).abs().sum().item() / h ** 0.5


@pytest.mark.parametrize("one_p", [False, True], ids=["plain", "1p"])
def test_mixed_fused_classes_match_torch(one_p):
    """MixedFusedLayerNorm / MixedFusedRMSNorm (megatron/model/fused_layer_norm.py:34-262) against torch's
    layer_norm / rms_norm on the same weights, including the zero-centred (`1p`) parameter storage."""
    from megatron.model.fused_layer_norm import MixedFusedLayerNorm, MixedFusedRMSNorm

    dtype, h = torch.bfloat16, 2048
    x = util.randn((48, 4, h), dtype, seed=5, std=2.0).to(DEV)
    g = util.randn((48, 4, h), dtype, seed=6).to(DEV)
    w = (1 + 0.3 * torch.randn(h, generator=torch.Generator().manual_seed(1))).to(dtype).to(DEV)
    bb = (0.2 * torch.randn(h, generator=torch.Generator().manual_seed(2))).to(dtype).to(DEV)
    lim = 2.0 ** -7

    ln = MixedFusedLayerNorm(h, eps=1e-5, apply_layernorm_1p=one_p).to(DEV).to(dtype)
    with torch.no_grad():
        ln.weight.copy_(w - 1 if one_p else w)
        ln.bias.copy_(bb)
    eff_w = (ln.weight.detach() + 1) if one_p else ln.weight.detach()
    xa = x.clone().requires_grad_(True)
    y = ln(xa)
    y.backward(g)
    xr = x.clone().requires_grad_(True)
    wr = eff_w.clone().requires_grad_(True)
    br = bb.clone().requires_grad_(True)
    ref = F.layer_norm(xr, (h,), wr, br, 1e-5)
    ref.backward(g)
    util.assert_close_ulp_or_noise(y.detach().cpu(), ref.detach().cpu(), 2, out_noise(eff_w.cpu(), x.cpu()), "layernorm y")
    assert (xa.grad.float() - xr.grad.float()).norm() <= lim * xr.grad.float().norm()
    assert (ln.weight.grad.float() - wr.grad.float()).norm() <= lim * wr.grad.float().norm()
    assert (ln.bias.grad.float() - br.grad.float()).norm() <= lim * br.grad.float().norm()

    rms = MixedFusedRMSNorm(h, eps=1e-5, apply_rmsnorm_1p=one_p).to(DEV).to(dtype)
    with torch.no_grad():
        rms.scale.copy_(w - 1 if one_p else w)
    eff_s = (rms.scale.detach() + 1) if one_p else rms.scale.detach()
    xa = x.clone().requires_grad_(True)
    y = rms(xa)
    y.backward(g)
    xr = x.float().requires_grad_(True)
    sr = eff_s.float().clone().requires_grad_(True)
    ref = F.rms_norm(xr, (h,), sr, 1e-5)
    ref.backward(g.float())
    util.assert_close_ulp_or_noise(y.detach().cpu(), ref.detach().to(dtype).cpu(), 2, out_noise(eff_s.cpu(), x.cpu()), "rmsnorm y")
    assert (xa.grad.float() - xr.grad).norm() <= lim * xr.grad.norm()
    assert (rms.scale.grad.float() - sr.grad).norm() <= lim * sr.grad.norm()


@pytest.mark.parametrize("cols", [2048, 2560, 5120, 6144], ids=lambda c: f"hidden{c}")
def test_layernorm_full_size(hotpath, cols):
    """The hidden state of the 1.4B configuration, [2048*8, 2048] bf16 with fp32 parameters, and the hidden sizes of
    the 2.8B, 12B and 20B configurations (workgroups of 3, 5 and 6 or 8 waves per row, a bounded grid that loops)."""
    rows = 2048 * 8
    gen = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn((rows, cols), generator=gen, device=DEV) * 2 + 0.5).bfloat16()
    dy = torch.randn((rows, cols), generator=gen, device=DEV).bfloat16()
    gamma = 1 + 0.3 * torch.randn(cols, generator=gen, device=DEV)
    beta = 0.2 * torch.randn(cols, generator=gen, device=DEV)
    y, mean, rstd, dx, dg, db = abi_layernorm(hotpath, x, dy, gamma, beta, 1e-5)
    pick = torch.tensor([0, 1, 3, 4, 4095, 9001, rows - 1], device=DEV)
    xc, dyc = x[pick].cpu(), dy[pick].cpu()
    want_y, _, _ = oracle.layernorm_fwd(xc, gamma.cpu(), beta.cpu(), 1e-5)
    util.assert_close_ulp_or_noise(y[pick].cpu(), want_y, 2, out_noise(gamma.cpu(), xc), "y rows")
    want_dx, _, _ = oracle.layernorm_bwd(dyc, xc, mean[pick].cpu(), rstd[pick].cpu(), gamma.cpu())
    util.assert_close_ulp_or_noise(dx[pick].cpu(), want_dx, 2, dx_noise(dyc, gamma.cpu(), rstd[pick].cpu()), "dx rows")
    xr = x.float().requires_grad_(True)
    gr = gamma.clone().requires_grad_(True)
    br = beta.clone().requires_grad_(True)
    F.layer_norm(xr, (cols,), gr, br, 1e-5).backward(dy.float())
    assert (dg - gr.grad).abs().max().item() <= 1e-3 * gr.grad.abs().max().item()
    assert (db - br.grad).abs().max().item() <= 1e-3 * br.grad.abs().max().item()
    assert (dx.float() - xr.grad).norm().item() <= 2.0**-8 * xr.grad.norm().item()


def test_layer_kernels_in_a_hip_graph_and_on_a_side_stream(hotpath):
    """LayerNorm forward + backward and bias+GeLU backward (each backward is two kernels that hand
    partial sums over through the caller's workspace) captured in one HIP graph: every replay, with
    eager work and synchronisation in between, gives the eager result bit for bit. The same calls
    on a non-default stream give the same bits as well."""
    L = hotpath.lib()
    rows, cols, BF16 = 777, 2048, hotpath.BF16
    x = torch.empty((rows, cols), dtype=torch.bfloat16, device=DEV)
    dy = util.randn((rows, cols), torch.bfloat16, seed=2).to(DEV)
    gamma = (1 + 0.3 * util.randn((cols,), torch.float32, seed=3)).bfloat16().to(DEV)
    beta = util.randn((cols,), torch.bfloat16, seed=4).to(DEV)

    def buffers():
        return dict(y=torch.empty_like(x), mean=torch.empty(rows, device=DEV), rstd=torch.empty(rows, device=DEV),
                    dx=torch.empty_like(x), dg=torch.empty_like(gamma), db=torch.empty_like(beta),
                    gx=torch.empty_like(x), gb=torch.empty_like(beta),
                    ws1=torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, BF16), 16), dtype=torch.uint8, device=DEV),
                    ws2=torch.empty(max(L.nhp_bias_gelu_bwd_workspace_bytes(rows, cols, BF16), 16), dtype=torch.uint8, device=DEV))

    def enqueue(b, st):
        assert L.nhp_layernorm_fwd(b["y"].data_ptr(), b["mean"].data_ptr(), b["rstd"].data_ptr(), x.data_ptr(), gamma.data_ptr(),
                                   beta.data_ptr(), 1e-5, rows, cols, BF16, BF16, st) == 0
        assert L.nhp_layernorm_bwd(b["dx"].data_ptr(), b["dg"].data_ptr(), b["db"].data_ptr(), dy.data_ptr(), x.data_ptr(),
                                   b["mean"].data_ptr(), b["rstd"].data_ptr(), gamma.data_ptr(), b["ws1"].data_ptr(), rows, cols,
                                   BF16, BF16, st) == 0
        assert L.nhp_bias_gelu_bwd(b["gx"].data_ptr(), dy.data_ptr(), x.data_ptr(), beta.data_ptr(), b["gb"].data_ptr(),
                                   b["ws2"].data_ptr(), rows, cols, BF16, st) == 0

    keys = ("y", "mean", "rstd", "dx", "dg", "db", "gx", "gb")
    captured, eager, aside = buffers(), buffers(), buffers()
    side = torch.cuda.Stream()
    x.copy_(util.randn((rows, cols), torch.bfloat16, seed=1, std=2.0).to(DEV))
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on a side stream, as capture needs
        enqueue(aside, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue(captured, torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        x.copy_(util.randn((rows, cols), torch.bfloat16, seed=10 + rep, std=2.0).to(DEV))
        for k in keys:
            captured[k].fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        enqueue(eager, None)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            enqueue(aside, side.cuda_stream)
        torch.cuda.synchronize()
        for k in keys:
            assert torch.equal(util.raw_bits(captured[k]), util.raw_bits(eager[k])), (rep, k)
            assert torch.equal(util.raw_bits(aside[k]), util.raw_bits(eager[k])), (rep, k)
