"""nhp_layernorm_bwd_noalloc (fixed device scratch array, no workspace argument, no allocation)
against nhp_layernorm_bwd (caller-provided workspace) through the C ABI.

Both entry points run the same kernels, so every output must be bit-identical. Two calls in a
row share the scratch array, the second on a smaller input: stale partial rows of the first
call must not leak into the second."""
import ctypes

import pytest
import torch

import util

DEV = "cuda"


def _inputs(dtype, rows, cols, seed, pdtype):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn((rows, cols), generator=g) * 2 + 0.5).to(dtype).to(DEV)
    dy = torch.randn((rows, cols), generator=g).to(dtype).to(DEV)
    gamma = (1 + 0.3 * torch.randn(cols, generator=g)).to(pdtype).to(DEV)
    beta = (0.2 * torch.randn(cols, generator=g)).to(pdtype).to(DEV)
    return x, dy, gamma, beta


def _stats(hp, x, gamma, beta):
    rows, cols = x.shape
    L = hp.lib()
    y = torch.empty_like(x)
    mean = torch.empty(rows, dtype=torch.float32, device=DEV)
    rstd = torch.empty_like(mean)
    rc = L.nhp_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), gamma.data_ptr(),
                             beta.data_ptr(), 1e-5, rows, cols, hp.dtype_code(x, "x"), hp._DTYPE[gamma.dtype], None)
    assert rc == 0, L.nhp_status_string(rc)
    return mean, rstd


def _backward(hp, noalloc, x, dy, gamma, mean, rstd):
    rows, cols = x.shape
    L = hp.lib()
    code, pcode = hp.dtype_code(x, "x"), hp._DTYPE[gamma.dtype]
    dx = torch.full_like(x, float("nan"))
    dg = torch.full_like(gamma, float("nan"))
    db = torch.full_like(gamma, float("nan"))
    if noalloc:
        rc = L.nhp_layernorm_bwd_noalloc(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                         mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(), rows, cols, code, pcode, None)
    else:
        ws = torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device=DEV)
        rc = L.nhp_layernorm_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                 mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(), ws.data_ptr(), rows, cols, code,
                                 pcode, None)
    assert rc == 0, L.nhp_status_string(rc)
    torch.cuda.synchronize()
    return dx, dg, db


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,pdtype", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32),
                                          (torch.float32, torch.float32)], ids=["bf16", "fp16-fp32params", "fp32"])
def test_noalloc_matches_workspace_entry_point_twice_in_a_row(hotpath, dtype, pdtype):
    hp = hotpath
    # a large call first, then a smaller one (fewer partial rows, shorter rows) on the same scratch array
    for rows, cols, seed in ((4096, 2048, 1), (300, 1000, 2)):
        x, dy, gamma, beta = _inputs(dtype, rows, cols, seed, pdtype)
        mean, rstd = _stats(hp, x, gamma, beta)
        want = _backward(hp, False, x, dy, gamma, mean, rstd)
        got = _backward(hp, True, x, dy, gamma, mean, rstd)
        for name, g, w in zip(("dx", "dgamma", "dbeta"), got, want):
            assert not torch.isnan(g.float()).any(), f"{name} not fully written ({rows}x{cols})"
            assert torch.equal(util.raw_bits(g), util.raw_bits(w)), f"{name} differs ({rows}x{cols})"


@pytest.mark.gpu
def test_noalloc_without_parameter_gradients_and_too_large(hotpath):
    hp = hotpath
    L = hp.lib()
    x, dy, gamma, beta = _inputs(torch.bfloat16, 512, 1024, 3, torch.bfloat16)
    mean, rstd = _stats(hp, x, gamma, beta)
    dx = torch.empty_like(x)
    rc = L.nhp_layernorm_bwd_noalloc(dx.data_ptr(), None, None, dy.data_ptr(), x.data_ptr(), mean.data_ptr(),
                                     rstd.data_ptr(), gamma.data_ptr(), 512, 1024, hp.BF16, hp.BF16, None)
    assert rc == 0
    want, _, _ = _backward(hp, False, x, dy, gamma, mean, rstd)
    torch.cuda.synchronize()
    assert torch.equal(util.raw_bits(dx), util.raw_bits(want))
    # rows so long that fewer than 8 pairs of partial rows fit the fixed array are refused before anything is launched
    rows, cols = 1 << 12, 1 << 19
    p = ctypes.c_void_p(0x1000)  # never dereferenced
    assert L.nhp_layernorm_bwd_noalloc(p, p, p, p, p, p, p, p, rows, cols, hp.BF16, hp.BF16, None) == -7


@pytest.mark.gpu
@pytest.mark.parametrize("cols", [5120, 6144, 8192])
def test_noalloc_with_fewer_partial_rows_than_the_workspace_entry_point(hotpath, cols):
    """At [16384, cols] beyond 4096 columns nhp_layernorm_bwd wants a workspace of more than 16 MiB
    (25-32 MiB): the entry point without allocation launches as many workgroups as have room for their
    partial rows in the fixed array. dx does not depend on the grid (bit-identical); dgamma / dbeta are the
    same column sums added in another order: within 2 ulp of the parameter dtype, or within the fp32
    rounding noise of a sum of that many terms."""
    hp = hotpath
    rows = 16384
    assert hp.lib().nhp_norm_bwd_workspace_bytes(rows, cols, hp.BF16) > 16 << 20
    for pdtype in (torch.bfloat16, torch.float32):
        x, dy, gamma, beta = _inputs(torch.bfloat16, rows, cols, 7, pdtype)
        mean, rstd = _stats(hp, x, gamma, beta)
        want = _backward(hp, False, x, dy, gamma, mean, rstd)
        got = _backward(hp, True, x, dy, gamma, mean, rstd)
        assert torch.equal(util.raw_bits(got[0]), util.raw_bits(want[0])), "dx"
        for name, g, w in zip(("dgamma", "dbeta"), got[1:], want[1:]):
            assert not torch.isnan(g.float()).any(), f"{name} not fully written"
            # |terms| of a column sum to about rows * E|dy * xhat| ~ rows; fp32 noise of re-ordering: a few eps of that
            noise = 8 * util.EPS32 * rows
            ok = (util.ulp_distance(g, w) <= 2) | ((g.float() - w.float()).abs() <= noise)
            assert bool(ok.all()), f"{name}: {int((~ok).sum())} columns differ beyond reordering noise"
