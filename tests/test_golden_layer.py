"""Committed golden vectors of the causal-softmax variants and the layer kernels
(tests/golden/layer_golden.npz, written by tests/golden/make_golden.py from the CPU
oracle). Without a GPU: the oracle reproduces them bit for bit. With a GPU: the HIP
path, called through the C ABI, matches them to the tolerance of the parity tests."""
import os

import numpy as np
import pytest
import torch

import oracle
import util

GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "layer_golden.npz"))
DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}
FP32_KEYS = ("slopes", "ln_mean", "ln_rstd", "rms0_inv", "rms1_inv", "part_inv", "sn_inv")


def get(prefix, key):
    arr = GOLDEN[f"{prefix}.{key}"]
    if arr.ndim == 0:
        return arr.item()
    t = torch.from_numpy(np.ascontiguousarray(arr))
    if key in ("lengths", "keep", "pad"):
        return t
    if key in FP32_KEYS:
        return t.view(torch.float32)
    return t.view(DT[prefix.split("_")[-1]])


def same(a, b):
    return torch.equal(util.raw_bits(a), util.raw_bits(b))


EX = ["ex_bf16", "ex_fp16"]
GELU = ["gelu_bf16", "gelu_fp16", "gelu_fp32"]
NORM = ["norm_bf16", "norm_fp16", "norm_fp32"]


@pytest.mark.parametrize("name", EX)
def test_oracle_reproduces_softmax_variant_golden(name):
    x, dy, bias, slopes, lengths = (get(name, k) for k in ("x", "dy", "bias", "slopes", "lengths"))
    window, scale = get(name, "window"), get(name, "scale")
    y = oracle.causal_softmax_fwd(x, scale, window=window, alibi_slopes=slopes, bias=bias, key_lengths=lengths)
    assert same(y, get(name, "y"))
    assert same(oracle.softmax_bwd(dy, y, scale, True, window=window, key_lengths=lengths), get(name, "dx"))


@pytest.mark.parametrize("name", GELU)
def test_oracle_reproduces_gelu_golden(name):
    y, bias, g, res = (get(name, k) for k in ("y", "bias", "g", "res"))
    assert same(oracle.bias_gelu_fwd(y, bias), get(name, "out"))
    dx = oracle.bias_gelu_bwd(g, y, bias)
    assert same(dx, get(name, "dx")) and same(oracle.column_sum(dx), get(name, "dbias"))
    assert same(oracle.bias_add_residual(y, bias, res), get(name, "added"))
    assert same(oracle.bias_add_residual_pair(y, bias, g, bias, res), get(name, "added_pair"))


@pytest.mark.parametrize("name", NORM)
def test_oracle_reproduces_norm_golden(name):
    x, dy, gamma, beta = (get(name, k) for k in ("x", "dy", "gamma", "beta"))
    y, mean, rstd = oracle.layernorm_fwd(x, gamma, beta, 1e-5)
    assert same(y, get(name, "ln_y")) and same(mean, get(name, "ln_mean")) and same(rstd, get(name, "ln_rstd"))
    dx, dg, db = oracle.layernorm_bwd(dy, x, mean, rstd, gamma)
    assert same(dx, get(name, "ln_dx")) and same(dg, get(name, "ln_dgamma")) and same(db, get(name, "ln_dbeta"))
    for mode in (0, 1):
        eps = get(name, f"rms{mode}_eps")
        ry, inv = oracle.rmsnorm_fwd(x, gamma, beta, eps, mode)
        assert same(ry, get(name, f"rms{mode}_y")) and same(inv, get(name, f"rms{mode}_inv"))
        rdx, rds, rdo = oracle.rmsnorm_bwd(dy, x, inv, gamma, eps, mode)
        assert same(rdx, get(name, f"rms{mode}_dx")) and same(rds, get(name, f"rms{mode}_dscale"))
        assert same(rdo, get(name, f"rms{mode}_doffset"))
    py, pinv = oracle.rmsnorm_fwd(x, gamma, beta, 1e-2, 1, stat_cols=7)
    assert same(py, get(name, "part_y")) and same(pinv, get(name, "part_inv"))
    pdx, pds, pdo = oracle.rmsnorm_bwd(dy, x, pinv, gamma, 1e-2, 1, stat_cols=7)
    assert same(pdx, get(name, "part_dx")) and same(pds, get(name, "part_dscale")) and same(pdo, get(name, "part_doffset"))
    gvec = torch.full((24,), 1.25, dtype=x.dtype)
    sy, sinv = oracle.rmsnorm_fwd(x, gvec, None, 1e-2, 2)
    assert same(sy, get(name, "sn_y")) and same(sinv, get(name, "sn_inv"))
    sdx, sds, _ = oracle.rmsnorm_bwd(dy, x, sinv, gvec, 1e-2, 2)
    assert same(sdx, get(name, "sn_dx")) and same(sds, get(name, "sn_dscale"))
    gamma2, beta2, dy2 = (get(name, k) for k in ("gamma2", "beta2", "dy2"))
    y1, y2, _, _ = oracle.layernorm_pair_fwd(x, gamma, beta, gamma2, beta2, 1e-5)
    assert same(y1, get(name, "ln_y")) and same(y2, get(name, "pair_y2"))
    pair = oracle.layernorm_pair_bwd(dy, dy2, x, mean, rstd, gamma, gamma2)
    assert same(pair[0], get(name, "pair_dx")) and same(pair[1], get(name, "ln_dgamma")) and same(pair[2], get(name, "ln_dbeta"))
    assert same(pair[3], get(name, "pair_dgamma2")) and same(pair[4], get(name, "pair_dbeta2"))


GATED = ["gated_bf16", "gated_fp16", "gated_fp32"]


@pytest.mark.parametrize("name", GATED)
def test_oracle_reproduces_gated_golden(name):
    inp, bias, dy = (get(name, k) for k in ("inp", "bias", "dy"))
    for act in sorted(oracle.GATE_ACTS):
        assert same(oracle.gated_act_fwd(inp, act, bias), get(name, f"{act}_out")), act
        assert same(oracle.gated_act_bwd(dy, inp, act, bias), get(name, f"{act}_din")), act


DROP = ["drop_bf16", "drop_fp16"]


@pytest.mark.parametrize("name", DROP)
def test_oracle_reproduces_dropout_golden(name):
    x, dy, bias = (get(name, k) for k in ("x", "dy", "bias"))
    p, seed, scale = get(name, "p"), get(name, "seed"), get(name, "scale")
    assert torch.equal(oracle.dropout_mask(x.numel(), p, seed).to(torch.uint8), get(name, "keep"))
    dropped, y = oracle.causal_softmax_dropout_fwd(x, scale, p, seed)
    assert same(y, get(name, "y")) and same(dropped, get(name, "dropped"))
    assert same(oracle.causal_softmax_dropout_bwd(dy, y, scale, p, seed), get(name, "dx"))
    assert same(oracle.bias_dropout_add(x.view(-1, 24), bias, dy.view(-1, 24), p, seed), get(name, "bda"))
    pad = get(name, "pad").bool()
    mdropped, my = oracle.masked_softmax_dropout_fwd(x.view(3, 1, 24, 24), pad, scale, p, seed)
    assert same(my, get(name, "m_y")) and same(mdropped, get(name, "m_dropped"))
    assert same(oracle.masked_softmax_dropout_bwd(dy.view(3, 1, 24, 24), my, scale, p, seed), get(name, "m_dx"))


def ptr(t):
    return None if t is None else t.data_ptr()


@pytest.mark.gpu
@pytest.mark.parametrize("name", DROP)
def test_gpu_matches_dropout_golden(hotpath, name):
    x, dy, bias, y = (get(name, k).cuda() for k in ("x", "dy", "bias", "y"))
    p, seed, scale = get(name, "p"), get(name, "seed"), get(name, "scale")
    L, code = hotpath.lib(), hotpath.dtype_code(x, "t")
    a, s = x.size(0), x.size(1)
    gy, gd = torch.empty_like(x), torch.empty_like(x)
    assert L.nhp_causal_softmax_dropout_fwd(gd.data_ptr(), gy.data_ptr(), x.data_ptr(), scale, a, s, -1, p, seed, 0, code, None) == 0
    util.assert_ulp_close(gy.cpu(), y.cpu(), 2, name)
    keep = get(name, "keep").view(a, s, s).bool()
    assert int(util.raw_bits(gd.cpu())[~keep].abs().max()) == 0                       # the golden mask, bit for bit
    assert same(gd.cpu(), oracle.bias_dropout_add(gy.cpu(), None, None, p, seed))     # dropout of the GPU's own y
    gdx = torch.empty_like(x)
    assert L.nhp_causal_softmax_dropout_bwd(gdx.data_ptr(), dy.data_ptr(), y.data_ptr(), scale, a, s, -1, p, seed, 0, code, None) == 0
    g = oracle.bias_dropout_add(dy.cpu(), None, None, p, seed)
    upper = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
    util.assert_softmax_bwd_close(gdx.cpu(), get(name, "dx"), g.masked_fill(upper, 0), y.cpu(), scale, name)
    out = torch.empty((a * s, s), dtype=x.dtype, device="cuda")
    assert L.nhp_bias_dropout_add(out.data_ptr(), x.data_ptr(), bias.data_ptr(), dy.data_ptr(), a * s, s, p, seed, 0, code, None) == 0
    assert same(out.cpu(), get(name, "bda"))
    # the padding-mask softmax with dropout
    pad = get(name, "pad").cuda()
    my, x4, dy4 = get(name, "m_y").cuda(), x.view(3, 1, s, s), dy.view(3, 1, s, s)
    assert L.nhp_masked_softmax_dropout_fwd(gd.data_ptr(), gy.data_ptr(), x4.data_ptr(), pad.data_ptr(), scale, 3, 1, s, s, 3, p, seed,
                                            0, code, None) == 0
    util.assert_ulp_close(gy.cpu().view(3, 1, s, s), my.cpu(), 2, name)
    assert same(gd.cpu(), oracle.bias_dropout_add(gy.cpu(), None, None, p, seed))
    assert L.nhp_masked_softmax_dropout_bwd(gdx.data_ptr(), dy4.data_ptr(), my.data_ptr(), scale, 3 * s, s, p, seed, 0, code, None) == 0
    util.assert_softmax_bwd_close(gdx.cpu(), get(name, "m_dx").view(3, s, s), g, my.cpu().view(3, s, s), scale, name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", GATED)
def test_gpu_matches_gated_golden(hotpath, name):
    inp, bias, dy = (get(name, k) for k in ("inp", "bias", "dy"))
    L, code = hotpath.lib(), hotpath.dtype_code(inp, "t")
    di, db, dd = inp.cuda(), bias.cuda(), dy.cuda()
    rows, f = dy.shape
    for act, num in sorted(oracle.GATE_ACTS.items()):
        out, din = torch.empty_like(dd), torch.empty_like(di)
        assert L.nhp_gated_act_fwd(out.data_ptr(), di.data_ptr(), db.data_ptr(), rows, f, num, code, None) == 0
        assert L.nhp_gated_act_bwd(din.data_ptr(), dd.data_ptr(), di.data_ptr(), db.data_ptr(), rows, f, num, code, None) == 0
        want, want_d = get(name, f"{act}_out"), get(name, f"{act}_din")
        util.assert_close_ulp_or_noise(out.cpu(), want, 2, util.gated_noise(inp, bias, act, want), f"{name} {act}")
        util.assert_close_ulp_or_noise(din.cpu(), want_d, 2, util.gated_noise(inp, bias, act, want_d, dy), f"{name} {act}")


@pytest.mark.gpu
@pytest.mark.parametrize("name", EX)
def test_gpu_matches_softmax_variant_golden(hotpath, name):
    x, dy, bias, slopes, lengths, y, dx = (get(name, k).cuda() for k in ("x", "dy", "bias", "slopes", "lengths", "y", "dx"))
    window, scale = get(name, "window"), get(name, "scale")
    L, code = hotpath.lib(), hotpath.dtype_code(x, "t")
    got = torch.empty_like(x)
    assert L.nhp_causal_softmax_ex_fwd(got.data_ptr(), x.data_ptr(), scale, x.size(0), x.size(1), window, slopes.data_ptr(),
                                       bias.data_ptr(), lengths.data_ptr(), 2, code, None) == 0
    zeros = util.raw_bits(y.cpu()) == 0
    assert int(util.raw_bits(got.cpu())[zeros & (y.cpu().float() == 0)].abs().max()) == 0
    util.assert_ulp_close(got.cpu(), y.cpu(), 2, name)
    gdx = torch.empty_like(x)
    assert L.nhp_causal_softmax_ex_bwd(gdx.data_ptr(), dy.data_ptr(), y.data_ptr(), scale, x.size(0), x.size(1), window,
                                       lengths.data_ptr(), 2, code, None) == 0
    util.assert_softmax_bwd_close(gdx.cpu(), dx.cpu(), dy.cpu() * (y.cpu() != 0), y.cpu(), scale, name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", GELU)
def test_gpu_matches_gelu_golden(hotpath, name):
    y, bias, g, res = (get(name, k).cuda() for k in ("y", "bias", "g", "res"))
    L, code = hotpath.lib(), hotpath.dtype_code(y, "t")
    rows, cols = y.shape
    x32 = (bias.float() + y.float()).cpu()
    out = torch.empty_like(y)
    assert L.nhp_bias_gelu_fwd(out.data_ptr(), y.data_ptr(), bias.data_ptr(), rows, cols, code, None) == 0
    util.assert_close_ulp_or_noise(out.cpu(), get(name, "out"), 2, util.gelu_noise(x32), name)
    dx, dbias = torch.empty_like(y), torch.empty_like(bias)
    ws = torch.empty(max(L.nhp_bias_gelu_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device="cuda")
    assert L.nhp_bias_gelu_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), bias.data_ptr(), dbias.data_ptr(), ws.data_ptr(),
                               rows, cols, code, None) == 0
    util.assert_close_ulp_or_noise(dx.cpu(), get(name, "dx"), 2, util.gelu_noise(x32, g.cpu()), name)
    util.assert_close_ulp_or_noise(dbias.cpu(), oracle.column_sum(dx.cpu()), 1, dx.float().abs().sum(0).cpu() * 16 * util.EPS32, name)
    added = torch.empty_like(y)
    assert L.nhp_bias_add_residual(added.data_ptr(), y.data_ptr(), bias.data_ptr(), res.data_ptr(), rows, cols, code, None) == 0
    assert same(added.cpu(), get(name, "added"))
    joined = torch.empty_like(added)
    assert L.nhp_bias_add_residual_pair(joined.data_ptr(), y.data_ptr(), bias.data_ptr(), g.data_ptr(), bias.data_ptr(),
                                        res.data_ptr(), rows, cols, code, None) == 0
    assert same(joined.cpu(), get(name, "added_pair"))


@pytest.mark.gpu
@pytest.mark.parametrize("name", NORM)
def test_gpu_matches_norm_golden(hotpath, name):
    x, dy, gamma, beta = (get(name, k).cuda() for k in ("x", "dy", "gamma", "beta"))
    L, code = hotpath.lib(), hotpath.dtype_code(x, "t")
    rows, cols = x.shape
    noise_y = (gamma.float().abs().cpu() * 64 * util.EPS32).expand(rows, cols)
    ws = torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device="cuda")

    def dx_noise(inv):
        return ((dy.float().abs() * gamma.float().abs()).sum(-1, keepdim=True).cpu() * inv[:, None] * 64 * util.EPS32).expand(rows, cols)

    col = dy.float().abs().sum(0).cpu() * 8 * 64 * util.EPS32
    y, mean, rstd = torch.empty_like(x), torch.empty(rows, device="cuda"), torch.empty(rows, device="cuda")
    assert L.nhp_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(),
                               1e-5, rows, cols, code, code, None) == 0
    util.assert_close_ulp_or_noise(y.cpu(), get(name, "ln_y"), 2, noise_y, name)
    assert torch.allclose(mean.cpu(), get(name, "ln_mean"), rtol=0, atol=1e-5)
    assert torch.allclose(rstd.cpu(), get(name, "ln_rstd"), rtol=1e-5, atol=0)
    gm, gr = get(name, "ln_mean").cuda(), get(name, "ln_rstd").cuda()
    dx, dg, db = torch.empty_like(x), torch.empty_like(gamma), torch.empty_like(beta)
    assert L.nhp_layernorm_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dy.data_ptr(), x.data_ptr(), gm.data_ptr(),
                               gr.data_ptr(), gamma.data_ptr(), ws.data_ptr(), rows, cols, code, code, None) == 0
    util.assert_close_ulp_or_noise(dx.cpu(), get(name, "ln_dx"), 2, dx_noise(gr.cpu()), name)
    util.assert_close_ulp_or_noise(dg.cpu(), get(name, "ln_dgamma"), 2, col, name)
    util.assert_close_ulp_or_noise(db.cpu(), get(name, "ln_dbeta"), 2, col, name)
    for mode in (0, 1):
        eps = get(name, f"rms{mode}_eps")
        inv = torch.empty(rows, device="cuda")
        assert L.nhp_rmsnorm_fwd(y.data_ptr(), inv.data_ptr(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), eps, mode,
                                 rows, cols, code, code, None) == 0
        util.assert_close_ulp_or_noise(y.cpu(), get(name, f"rms{mode}_y"), 2, noise_y, name)
        gi = get(name, f"rms{mode}_inv").cuda()
        assert torch.allclose(inv.cpu(), gi.cpu(), rtol=1e-5, atol=0)
        assert L.nhp_rmsnorm_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dy.data_ptr(), x.data_ptr(), gi.data_ptr(),
                                 gamma.data_ptr(), ws.data_ptr(), eps, mode, rows, cols, code, code, None) == 0
        util.assert_close_ulp_or_noise(dx.cpu(), get(name, f"rms{mode}_dx"), 2, dx_noise(gi.cpu()), name)
        util.assert_close_ulp_or_noise(dg.cpu(), get(name, f"rms{mode}_dscale"), 2, col, name)
        util.assert_close_ulp_or_noise(db.cpu(), get(name, f"rms{mode}_doffset"), 2, col, name)
    # partial RMSNorm and ScaleNorm
    inv = torch.empty(rows, device="cuda")
    assert L.nhp_rmsnorm_partial_fwd(y.data_ptr(), inv.data_ptr(), x.data_ptr(), gamma.data_ptr(), beta.data_ptr(), 1e-2, 1,
                                     rows, cols, 7, code, code, None) == 0
    grow = (get(name, "x").float().abs() * get(name, "part_inv")[:, None]).clamp(min=1.0)
    util.assert_close_ulp_or_noise(y.cpu(), get(name, "part_y"), 2, noise_y * grow, name)
    gi = get(name, "part_inv").cuda()
    assert torch.allclose(inv.cpu(), gi.cpu(), rtol=1e-5, atol=0)
    assert L.nhp_rmsnorm_partial_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dy.data_ptr(), x.data_ptr(), gi.data_ptr(),
                                     gamma.data_ptr(), ws.data_ptr(), 1e-2, 1, rows, cols, 7, code, code, None) == 0
    util.assert_close_ulp_or_noise(dx.cpu(), get(name, "part_dx"), 2, dx_noise(gi.cpu()) * grow * cols / 7, name)
    util.assert_close_ulp_or_noise(dg.cpu(), get(name, "part_dscale"), 2, col * grow.amax(0), name)
    util.assert_close_ulp_or_noise(db.cpu(), get(name, "part_doffset"), 2, col, name)
    gvec = torch.full((cols,), 1.25, dtype=x.dtype, device="cuda")
    assert L.nhp_rmsnorm_fwd(y.data_ptr(), inv.data_ptr(), x.data_ptr(), gvec.data_ptr(), None, 1e-2, 2, rows, cols, code,
                             code, None) == 0
    util.assert_close_ulp_or_noise(y.cpu(), get(name, "sn_y"), 2, noise_y, name)
    gi = get(name, "sn_inv").cuda()
    assert torch.allclose(inv.cpu(), gi.cpu(), rtol=1e-5, atol=0)
    assert L.nhp_rmsnorm_bwd(dx.data_ptr(), dg.data_ptr(), None, dy.data_ptr(), x.data_ptr(), gi.data_ptr(), gvec.data_ptr(),
                             ws.data_ptr(), 1e-2, 2, rows, cols, code, code, None) == 0
    util.assert_close_ulp_or_noise(dx.cpu(), get(name, "sn_dx"), 2, dx_noise(gi.cpu()) * 2, name)
    util.assert_close_ulp_or_noise(dg.cpu(), get(name, "sn_dscale"), 2, col, name)

    # two LayerNorms of one input
    gamma2, beta2, dy2 = (get(name, k).cuda() for k in ("gamma2", "beta2", "dy2"))
    y2 = torch.empty_like(x)
    assert L.nhp_layernorm_pair_fwd(y.data_ptr(), y2.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(),
                                    gamma.data_ptr(), beta.data_ptr(), gamma2.data_ptr(), beta2.data_ptr(), 1e-5, rows, cols,
                                    code, code, None) == 0
    util.assert_close_ulp_or_noise(y.cpu(), get(name, "ln_y"), 2, noise_y, name)
    util.assert_close_ulp_or_noise(y2.cpu(), get(name, "pair_y2"), 2, (gamma2.float().abs().cpu() * 64 * util.EPS32).expand(rows, cols), name)
    ws2 = torch.empty(max(L.nhp_layernorm_pair_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device="cuda")
    dg2, db2 = torch.empty_like(gamma), torch.empty_like(beta)
    gm, gr = get(name, "ln_mean").cuda(), get(name, "ln_rstd").cuda()
    assert L.nhp_layernorm_pair_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dg2.data_ptr(), db2.data_ptr(), dy.data_ptr(),
                                    dy2.data_ptr(), x.data_ptr(), gm.data_ptr(), gr.data_ptr(), gamma.data_ptr(),
                                    gamma2.data_ptr(), ws2.data_ptr(), rows, cols, code, code, None) == 0
    both = ((dy.float().abs() * gamma.float().abs() + dy2.float().abs() * gamma2.float().abs()).sum(-1, keepdim=True).cpu()
            * gr.cpu()[:, None] * 64 * util.EPS32).expand(rows, cols)
    util.assert_close_ulp_or_noise(dx.cpu(), get(name, "pair_dx"), 2, both, name)
    col2 = dy2.float().abs().sum(0).cpu() * 8 * 64 * util.EPS32
    util.assert_close_ulp_or_noise(dg.cpu(), get(name, "ln_dgamma"), 2, col, name)
    util.assert_close_ulp_or_noise(db.cpu(), get(name, "ln_dbeta"), 2, col, name)
    util.assert_close_ulp_or_noise(dg2.cpu(), get(name, "pair_dgamma2"), 2, col2, name)
    util.assert_close_ulp_or_noise(db2.cpu(), get(name, "pair_dbeta2"), 2, col2, name)