"""Randomised differential test: every kernel family against the CPU oracle on shapes drawn
around the boundaries of the launch geometries (multiples of the 16-byte chunk +-1, powers
of two +-8, one row, one column, rows that end in the middle of a workgroup). Seeds are fixed:
the cases are the same on every run. Tolerances as in the per-kernel parity tests."""
import math
import random

import pytest
import torch

import oracle
import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"
HALF = [torch.bfloat16, torch.float16]
ALL = HALF + [torch.float32]


def boundary_int(rng, lo, hi):
    """An integer in [lo, hi], biased towards chunk and power-of-two boundaries."""
    kind = rng.random()
    if kind < 0.35:
        v = (1 << rng.randint(0, max(0, hi.bit_length() - 1))) + rng.choice((-8, -1, 0, 1, 8))
    elif kind < 0.7:
        v = 8 * rng.randint(1, max(1, hi // 8)) + rng.choice((-1, 0, 0, 1))
    else:
        v = rng.randint(lo, hi)
    return max(lo, min(hi, v))


def ptr(t):
    return None if t is None else t.data_ptr()


@pytest.mark.parametrize("seed", range(24))
def test_causal_softmax_random_shapes(hotpath, seed):
    import scaled_upper_triang_masked_softmax_cuda as ext

    rng = random.Random(1000 + seed)
    dtype = rng.choice(HALF)
    a, s = rng.randint(1, 5), boundary_int(rng, 1, 1500)
    window = rng.choice((None, None, rng.randint(0, s)))
    scale = rng.choice((1.0, 0.125, 1 / math.sqrt(128), 0.3))
    print(f"causal a={a} s={s} window={window} {dtype} scale={scale}", flush=True)
    x = util.randn((a, s, s), dtype, seed=seed, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=seed + 1)
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    want = oracle.causal_softmax_fwd(x, scale, window=window)
    got = ext.forward(x.to(DEV), scale, window).cpu()
    if masked.any():
        assert int(util.raw_bits(got)[:, masked].abs().max()) == 0
    util.assert_ulp_close(got, want, 2, "fwd")
    want_dx = oracle.softmax_bwd(dy, want, scale, True, window=window)
    got_dx = ext.backward(dy.to(DEV).clone(), want.to(DEV), scale, window).cpu()
    util.assert_softmax_bwd_close(got_dx, want_dx, dy.masked_fill(masked, 0), want, scale, "bwd")
    if rng.random() < 0.5:
        p, sd = rng.choice((0.1, 0.5)), rng.randint(0, 1 << 40)
        dropped, y = [t.cpu() for t in ext.forward_dropout(x.to(DEV), scale, p, sd, window)]
        util.assert_ulp_close(y, want, 2, "dropout y")
        assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(y, None, None, p, sd)))


@pytest.mark.parametrize("seed", range(16))
def test_masked_softmax_random_shapes(hotpath, seed):
    rng = random.Random(2000 + seed)
    dtype = rng.choice(HALF)
    b, np_, sq, sk = rng.randint(1, 3), rng.randint(1, 5), rng.randint(2, 9), boundary_int(rng, 1, 3000)
    pb = rng.choice((1, b))
    scale = rng.choice((1.0, 0.125, 1 / math.sqrt(128)))
    print(f"masked b={b} np={np_} sq={sq} sk={sk} pb={pb} {dtype}", flush=True)
    x = util.randn((b, np_, sq, sk), dtype, seed=seed, std=3.0)
    dy = util.randn((b, np_, sq, sk), dtype, seed=seed + 1)
    mask = util.padding_mask(pb, sq, sk, seed, full_batch=0 if rng.random() < 0.3 else None)
    want = oracle.masked_softmax_fwd(x, mask, scale)
    got = util.abi_masked_fwd(hotpath, x.to(DEV), mask.to(DEV), scale).cpu()
    util.assert_ulp_close(got, want, 2, "fwd")
    want_dx = oracle.softmax_bwd(dy, want, scale, False)
    got_dx = util.abi_masked_bwd(hotpath, dy.to(DEV), want.to(DEV), scale).cpu()
    util.assert_softmax_bwd_close(got_dx, want_dx, dy, want, scale, "bwd")
    if rng.random() < 0.6:   # the same with attention dropout in the kernel
        import scaled_masked_softmax_cuda as ext

        p, sd = rng.choice((0.1, 0.5)), rng.randint(0, 1 << 40)
        if sq > 1:
            dropped, y = [t.cpu() for t in ext.forward_dropout(x.to(DEV), mask.to(DEV), scale, p, sd)]
            util.assert_ulp_close(y, want, 2, "fwd with dropout")
            assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(y, None, None, p, sd)))
            got_ddx = ext.backward_dropout(dy.to(DEV).clone(), want.to(DEV), scale, p, sd).cpu()
            g = oracle.bias_dropout_add(dy, None, None, p, sd)
            util.assert_softmax_bwd_close(got_ddx, oracle.masked_softmax_dropout_bwd(dy, want, scale, p, sd), g, want, scale,
                                          "bwd with dropout")


@pytest.mark.parametrize("seed", range(16))
def test_rope_random_shapes(hotpath, seed):
    rng = random.Random(3000 + seed)
    dtype = rng.choice(ALL)
    s, b, h = rng.randint(1, 40), rng.randint(1, 3), rng.randint(1, 5)
    d = rng.choice((8, 16, 24, 32, 64, 96, 128, 256, 20, 6))
    d2 = rng.choice([v for v in (d, d // 2, d // 4, 2, 4, 8) if 2 <= v <= d and v % 2 == 0])
    print(f"rope s={s} b={b} h={h} d={d} d2={d2} {dtype}", flush=True)
    t = util.randn((s, b, h, d), dtype, seed=seed)
    g = torch.Generator().manual_seed(seed)
    ang = (torch.rand((s, 1, 1, d2), generator=g) * 20 - 10).contiguous()
    cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)
    for backward in (False, True):
        want = oracle.rope_cached(t, cos, sin, backward=backward)
        got = util.abi_rope_cached(hotpath, t.to(DEV), cos.to(DEV), sin.to(DEV), backward=backward).cpu()
        assert torch.equal(util.raw_bits(got), util.raw_bits(want)), backward
    # the same values laid out contiguously along the sequence (the layout of the key gradient)
    seq_major = t.permute(1, 2, 3, 0).contiguous().to(DEV).permute(3, 0, 1, 2)
    assert seq_major.stride(0) == 1 or s == 1
    for backward in (False, True):
        want = oracle.rope_cached(t, cos, sin, backward=backward)
        got = util.abi_rope_cached(hotpath, seq_major, cos.to(DEV), sin.to(DEV), backward=backward).cpu()
        assert torch.equal(util.raw_bits(got), util.raw_bits(want)), ("sequence-major", backward)


@pytest.mark.parametrize("seed", range(24))
def test_rope_two_tensor_launches_random_shapes(hotpath, seed):
    """q and k through the two-tensor entry points in the layouts a caller may hand over: separate tensors, slices
    of one buffer along the heads (k possibly with fewer heads), slices along the features in the order of a fused
    projection (k directly behind q: read as one run per row) or in another order, both output layouts, both
    table sources. Bit-exact against the oracle (cached tables) or the single-tensor entry point (angles)."""
    rng = random.Random(3300 + seed)
    dtype = rng.choice(ALL)
    s, b, h = rng.randint(1, 40), rng.randint(1, 3), rng.randint(1, 6)
    d = rng.choice((8, 16, 32, 64, 96, 128, 256, 80, 24))
    d2 = rng.choice([v for v in (d, d // 2, d // 4, 8, 6) if 2 <= v <= d and v % 2 == 0])
    layout = rng.choice(("separate", "heads", "features", "features-reversed", "features-gap"))
    hk = h
    if layout == "separate":
        hk = rng.randint(1, h)
        q = util.randn((s, b, h, d), dtype, seed=seed).to(DEV)
        k = util.randn((s, b, hk, d), dtype, seed=seed + 50).to(DEV)
    elif layout == "heads":
        hk = rng.randint(1, h)
        buf = util.randn((s, b, h + 2 * hk, d), dtype, seed=seed).to(DEV)
        q, k = buf[:, :, :h], buf[:, :, h:h + hk]
    else:
        buf = util.randn((s, b, h, 4 * d), dtype, seed=seed).to(DEV)
        if layout == "features":
            q, k = buf[..., :d], buf[..., d:2 * d]
        elif layout == "features-reversed":
            q, k = buf[..., d:2 * d], buf[..., :d]
        else:
            q, k = buf[..., :d], buf[..., 2 * d:3 * d]
    transpose = rng.random() < 0.4
    print(f"rope two tensors s={s} b={b} h={h} hk={hk} d={d} d2={d2} {dtype} {layout} transpose={transpose}", flush=True)
    g = torch.Generator().manual_seed(seed)
    ang = (torch.rand((s, 1, 1, d2), generator=g) * 20 - 10).contiguous()
    cs = torch.float32 if rng.random() < 0.3 else dtype
    cos, sin = ang.cos().to(cs), ang.sin().to(cs)
    cos_d, sin_d, ang_d = cos.to(DEV), sin.to(DEV), ang.to(DEV)
    L = hotpath.lib()
    code = hotpath.dtype_code(q, "t")
    for backward in (False, True):
        got_q, got_k = util._rope_out(q, transpose), util._rope_out(k, transpose)
        fn = L.nhp_rope_cached_qk_bwd if backward else L.nhp_rope_cached_qk_fwd
        rc = fn(got_q.data_ptr(), got_k.data_ptr(), q.data_ptr(), k.data_ptr(), cos_d.data_ptr(), sin_d.data_ptr(), s, b, h, hk,
                d, d2, hotpath.strides4(q), hotpath.strides4(k), hotpath.strides4(got_q), hotpath.strides4(got_k), code,
                hotpath.dtype_code(cos_d, "c"), None)
        assert rc == 0, L.nhp_status_string(rc)
        torch.cuda.synchronize()
        assert torch.equal(util.raw_bits(got_q.cpu()), util.raw_bits(oracle.rope_cached(q.cpu(), cos, sin, backward, transpose)))
        assert torch.equal(util.raw_bits(got_k.cpu()), util.raw_bits(oracle.rope_cached(k.cpu(), cos, sin, backward, transpose)))
        got_q, got_k = util._rope_out(q, transpose), util._rope_out(k, transpose)
        fn = L.nhp_rope_freqs_qk_bwd if backward else L.nhp_rope_freqs_qk_fwd
        rc = fn(got_q.data_ptr(), got_k.data_ptr(), q.data_ptr(), k.data_ptr(), ang_d.data_ptr(), s, b, h, hk, d, d2,
                hotpath.strides4(q), hotpath.strides4(k), hotpath.strides4(got_q), hotpath.strides4(got_k), code, None)
        assert rc == 0, L.nhp_status_string(rc)
        torch.cuda.synchronize()
        assert torch.equal(util.raw_bits(got_q.cpu()), util.raw_bits(util.abi_rope_freqs(hotpath, q, ang_d, backward, transpose).cpu()))
        assert torch.equal(util.raw_bits(got_k.cpu()), util.raw_bits(util.abi_rope_freqs(hotpath, k, ang_d, backward, transpose).cpu()))


@pytest.mark.parametrize("seed", range(12))
def test_rope_sequence_major_random_shapes(hotpath, seed):
    """Shapes inside and around the conditions of the transposing kernel (s a multiple of 8 or not, every head
    size it takes and some it does not, windows of a longer sequence)."""
    rng = random.Random(3500 + seed)
    dtype = rng.choice(HALF)
    s_total = rng.choice((8, 64, 72, 200, 256, 1000, 1001, 130))
    b, h = rng.randint(1, 3), rng.randint(1, 5)
    d = rng.choice((32, 64, 80, 96, 128, 160, 256, 512, 24))
    d2 = rng.choice([v for v in (d, d // 2, d // 4, 16, 32) if 2 <= v <= d and v % 2 == 0])
    first = rng.choice((0, 0, 8, 3))
    s = s_total - first
    print(f"rope sequence-major s={s} of {s_total} b={b} h={h} d={d} d2={d2} {dtype}", flush=True)
    base = util.randn((b, h, d, s_total), dtype, seed=seed)
    t = base.permute(3, 0, 1, 2)[first:]
    t_d = base.to(DEV).permute(3, 0, 1, 2)[first:]
    g = torch.Generator().manual_seed(seed)
    ang = (torch.rand((s, 1, 1, d2), generator=g) * 20 - 10).contiguous()
    cs = torch.float32 if rng.random() < 0.3 else dtype
    cos, sin = ang.cos().to(cs), ang.sin().to(cs)
    for backward in (False, True):
        want = oracle.rope_cached(t.contiguous(), cos, sin, backward=backward)
        got = util.abi_rope_cached(hotpath, t_d, cos.to(DEV), sin.to(DEV), backward=backward).cpu()
        assert torch.equal(util.raw_bits(got), util.raw_bits(want)), backward


@pytest.mark.parametrize("seed", range(24))
def test_layer_kernels_random_shapes(hotpath, seed):
    rng = random.Random(4000 + seed)
    dtype = rng.choice(ALL)
    rows, cols = boundary_int(rng, 1, 600), boundary_int(rng, 1, 5000)
    L, code = hotpath.lib(), hotpath._DTYPE[dtype]
    print(f"layer rows={rows} cols={cols} {dtype}", flush=True)
    x = util.randn((rows, cols), dtype, seed=seed, std=2.5) + 0.25
    g = util.randn((rows, cols), dtype, seed=seed + 1)
    bias = util.randn((cols,), dtype, seed=seed + 2, std=0.5)
    gamma = (1 + 0.3 * util.randn((cols,), torch.float32, seed=seed + 3)).to(dtype)
    xd, gd, bd, gmd = x.to(DEV), g.to(DEV), bias.to(DEV), gamma.to(DEV)
    # bias + GeLU forward / backward with the bias gradient
    x32 = bias.float() + x.float()
    out, dx, dbias = torch.empty_like(xd), torch.empty_like(xd), torch.empty_like(bd)
    ws = torch.empty(max(L.nhp_bias_gelu_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device=DEV)
    assert L.nhp_bias_gelu_fwd(out.data_ptr(), xd.data_ptr(), bd.data_ptr(), rows, cols, code, None) == 0
    util.assert_close_ulp_or_noise(out.cpu(), oracle.bias_gelu_fwd(x, bias), 2, util.gelu_noise(x32), "gelu fwd")
    assert L.nhp_bias_gelu_bwd(dx.data_ptr(), gd.data_ptr(), xd.data_ptr(), bd.data_ptr(), dbias.data_ptr(), ws.data_ptr(), rows,
                               cols, code, None) == 0
    util.assert_close_ulp_or_noise(dx.cpu(), oracle.bias_gelu_bwd(g, x, bias), 2, util.gelu_noise(x32, g), "gelu bwd")
    util.assert_close_ulp_or_noise(dbias.cpu(), oracle.column_sum(dx.cpu()), 1, dx.float().abs().sum(0).cpu() * 16 * util.EPS32, "dbias")
    # bias + residual add, with and without dropout: bit-exact
    assert L.nhp_bias_add_residual(out.data_ptr(), xd.data_ptr(), bd.data_ptr(), gd.data_ptr(), rows, cols, code, None) == 0
    assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(oracle.bias_add_residual(x, bias, g)))
    p, sd = rng.choice((0.1, 0.5)), rng.randint(0, 1 << 50)
    assert L.nhp_bias_dropout_add(out.data_ptr(), xd.data_ptr(), bd.data_ptr(), gd.data_ptr(), rows, cols, p, sd, 3, code, None) == 0
    assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(oracle.bias_dropout_add(x, bias, g, p, sd, 3)))
    # LayerNorm and RMSNorm forward / backward
    nws = torch.empty(max(L.nhp_norm_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device=DEV)
    y, mean, rstd = torch.empty_like(xd), torch.empty(rows, device=DEV), torch.empty(rows, device=DEV)
    dg, db = torch.empty_like(gmd), torch.empty_like(gmd)
    noise_y = (gamma.float().abs() * 64 * util.EPS32).expand(rows, cols)
    assert L.nhp_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), xd.data_ptr(), gmd.data_ptr(), bd.data_ptr(), 1e-5,
                               rows, cols, code, code, None) == 0
    want_y, _, _ = oracle.layernorm_fwd(x, gamma, bias, 1e-5)
    util.assert_close_ulp_or_noise(y.cpu(), want_y, 2, noise_y, "layernorm fwd")
    assert L.nhp_layernorm_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), gd.data_ptr(), xd.data_ptr(), mean.data_ptr(),
                               rstd.data_ptr(), gmd.data_ptr(), nws.data_ptr(), rows, cols, code, code, None) == 0
    want_dx, want_dg, want_db = oracle.layernorm_bwd(g, x, mean.cpu(), rstd.cpu(), gamma)
    dxn = ((g.float().abs() * gamma.float().abs()).sum(-1, keepdim=True) * rstd.cpu()[:, None] * 64 * util.EPS32).expand(rows, cols)
    util.assert_close_ulp_or_noise(dx.cpu(), want_dx, 2, dxn, "layernorm dx")
    xhat = ((x.float() - mean.cpu()[:, None]) * rstd.cpu()[:, None]).abs()
    util.assert_close_ulp_or_noise(dg.cpu(), want_dg, 2, (g.float().abs() * xhat).sum(0) * 32 * util.EPS32, "dgamma")
    util.assert_close_ulp_or_noise(db.cpu(), want_db, 2, g.float().abs().sum(0) * 32 * util.EPS32, "dbeta")
    mode = rng.choice((0, 1))
    inv = torch.empty(rows, device=DEV)
    assert L.nhp_rmsnorm_fwd(y.data_ptr(), inv.data_ptr(), xd.data_ptr(), gmd.data_ptr(), None, 1e-5, mode, rows, cols, code, code,
                             None) == 0
    want_r, _ = oracle.rmsnorm_fwd(x, gamma, None, 1e-5, mode)
    util.assert_close_ulp_or_noise(y.cpu(), want_r, 2, noise_y, "rmsnorm fwd")
    # partial statistic (any number of leading columns) and the clamped-norm definition, forward and backward
    stat = rng.randint(1, cols)
    pmode = rng.choice((0, 1, 2))
    assert L.nhp_rmsnorm_partial_fwd(y.data_ptr(), inv.data_ptr(), xd.data_ptr(), gmd.data_ptr(), None, 1e-3, pmode, rows, cols,
                                     stat, code, code, None) == 0
    want_p, want_inv = oracle.rmsnorm_fwd(x, gamma, None, 1e-3, pmode, stat_cols=stat)
    grow = (x.float().abs() * want_inv[:, None]).clamp(min=1.0)
    util.assert_close_ulp_or_noise(y.cpu(), want_p, 2, noise_y * grow, f"partial rmsnorm fwd, stat {stat} mode {pmode}")
    assert torch.allclose(inv.cpu(), want_inv, rtol=1e-5, atol=0)
    assert L.nhp_rmsnorm_partial_bwd(dx.data_ptr(), dg.data_ptr(), None, gd.data_ptr(), xd.data_ptr(), inv.data_ptr(),
                                     gmd.data_ptr(), nws.data_ptr(), 1e-3, pmode, rows, cols, stat, code, code, None) == 0
    icpu = inv.cpu()
    want_pdx, want_pds, _ = oracle.rmsnorm_bwd(g, x, icpu, gamma, 1e-3, pmode, stat_cols=stat)
    xh = (x.float() * icpu[:, None]).abs()
    denom = 1.0 if pmode == 2 else float(stat)
    pnoise = ((g.float().abs() * gamma.float().abs() * xh).sum(-1, keepdim=True) * xh * icpu[:, None] / denom * 256 * util.EPS32
              + (g.float().abs() * gamma.float().abs()) * icpu[:, None] * 16 * util.EPS32)
    util.assert_close_ulp_or_noise(dx.cpu(), want_pdx, 2, pnoise, f"partial rmsnorm dx, stat {stat} mode {pmode}")
    util.assert_close_ulp_or_noise(dg.cpu(), want_pds, 2, (g.float().abs() * xh).sum(0) * 32 * util.EPS32, "partial rmsnorm dscale")
    # gated activation on the same data when the width is even
    if cols % 2 == 0:
        act = rng.choice(sorted(oracle.GATE_ACTS))
        f = cols // 2
        go = torch.empty((rows, f), dtype=dtype, device=DEV)
        assert L.nhp_gated_act_fwd(go.data_ptr(), xd.data_ptr(), bd.data_ptr(), rows, f, oracle.GATE_ACTS[act], code, None) == 0
        want_g = oracle.gated_act_fwd(x, act, bias)
        util.assert_close_ulp_or_noise(go.cpu(), want_g, 2, util.gated_noise(x, bias, act, want_g), f"gated {act}")


@pytest.mark.parametrize("seed", range(16))
def test_pair_kernels_random_shapes(hotpath, seed):
    """The two kernels of the parallel-residual layer: two LayerNorms of one input (forward and backward) and the
    join of the two branches with the residual, on boundary shapes."""
    rng = random.Random(6000 + seed)
    dtype = rng.choice(ALL)
    rows, cols = boundary_int(rng, 1, 400), boundary_int(rng, 1, 5000)
    pdtype = rng.choice((dtype, torch.float32))
    L, code, pcode = hotpath.lib(), hotpath._DTYPE[dtype], hotpath._DTYPE[pdtype]
    print(f"pair rows={rows} cols={cols} {dtype} params {pdtype}", flush=True)
    x = util.randn((rows, cols), dtype, seed=seed, std=2.5) + 0.25
    g1, g2 = (util.randn((rows, cols), dtype, seed=seed + 1 + i) for i in range(2))
    gam1, gam2 = ((1 + 0.3 * util.randn((cols,), torch.float32, seed=seed + 3 + i)).to(pdtype) for i in range(2))
    bet1, bet2 = ((0.2 * util.randn((cols,), torch.float32, seed=seed + 5 + i)).to(pdtype) for i in range(2))
    dev = {k: v.to(DEV) for k, v in dict(x=x, g1=g1, g2=g2, gam1=gam1, gam2=gam2, bet1=bet1, bet2=bet2).items()}
    # join of the branches: bit-exact, with a random choice of missing biases
    b1 = util.randn((cols,), dtype, seed=seed + 7) if rng.random() < 0.7 else None
    b2 = util.randn((cols,), dtype, seed=seed + 8) if rng.random() < 0.7 else None
    d1, d2 = (None if b is None else b.to(DEV) for b in (b1, b2))
    out = torch.empty_like(dev["x"])
    assert L.nhp_bias_add_residual_pair(out.data_ptr(), dev["x"].data_ptr(), ptr(d1), dev["g1"].data_ptr(), ptr(d2),
                                        dev["g2"].data_ptr(), rows, cols, code, None) == 0
    assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(oracle.bias_add_residual_pair(x, b1, g1, b2, g2)))
    # two LayerNorms of one input
    y1, y2, dx = (torch.empty_like(dev["x"]) for _ in range(3))
    mean, rstd = torch.empty(rows, device=DEV), torch.empty(rows, device=DEV)
    grads = [torch.empty_like(dev["gam1"]) for _ in range(4)]
    ws = torch.empty(max(L.nhp_layernorm_pair_bwd_workspace_bytes(rows, cols, code), 16), dtype=torch.uint8, device=DEV)
    assert L.nhp_layernorm_pair_fwd(y1.data_ptr(), y2.data_ptr(), mean.data_ptr(), rstd.data_ptr(), dev["x"].data_ptr(),
                                    dev["gam1"].data_ptr(), dev["bet1"].data_ptr(), dev["gam2"].data_ptr(),
                                    dev["bet2"].data_ptr(), 1e-5, rows, cols, code, pcode, None) == 0
    w1, w2, _, _ = oracle.layernorm_pair_fwd(x, gam1, bet1, gam2, bet2, 1e-5)
    for got, want, gam in ((y1, w1, gam1), (y2, w2, gam2)):
        util.assert_close_ulp_or_noise(got.cpu(), want, 2, (gam.float().abs() * 64 * util.EPS32).expand(rows, cols), "pair fwd")
    assert L.nhp_layernorm_pair_bwd(dx.data_ptr(), grads[0].data_ptr(), grads[1].data_ptr(), grads[2].data_ptr(),
                                    grads[3].data_ptr(), dev["g1"].data_ptr(), dev["g2"].data_ptr(), dev["x"].data_ptr(),
                                    mean.data_ptr(), rstd.data_ptr(), dev["gam1"].data_ptr(), dev["gam2"].data_ptr(),
                                    ws.data_ptr(), rows, cols, code, pcode, None) == 0
    mc, rc = mean.cpu(), rstd.cpu()
    want = oracle.layernorm_pair_bwd(g1, g2, x, mc, rc, gam1, gam2)
    noise = (((g1.float().abs() * gam1.float().abs() + g2.float().abs() * gam2.float().abs()).sum(-1, keepdim=True))
             * rc[:, None] * 64 * util.EPS32).expand(rows, cols)
    util.assert_close_ulp_or_noise(dx.cpu(), want[0], 2, noise, "pair dx")
    xhat = ((x.float() - mc[:, None]) * rc[:, None]).abs()
    for i, g in ((0, g1), (2, g2)):
        util.assert_close_ulp_or_noise(grads[i].cpu(), want[1 + i], 2, (g.float().abs() * xhat).sum(0) * 32 * util.EPS32, "dgamma")
        util.assert_close_ulp_or_noise(grads[i + 1].cpu(), want[2 + i], 2, g.float().abs().sum(0) * 32 * util.EPS32, "dbeta")


@pytest.mark.parametrize("seed", range(16))
def test_block_limited_softmax_random_shapes(hotpath, seed):
    """The causal softmax that writes only the blocks in use: random sequence length, window and block size; values
    inside the written range against the oracle, a sentinel outside of it."""
    import scaled_upper_triang_masked_softmax_cuda as ext
    from megatron.model.fused_softmax import _written_blocks

    rng = random.Random(7000 + seed)
    dtype = rng.choice(HALF)
    s = 8 * boundary_int(rng, 3, 300)
    a = rng.randint(1, 3)
    zb = 1 << rng.randint(3, 10)
    window = rng.choice((None, None, rng.randint(0, s + 10)))
    scale = rng.choice((1.0, 0.125, 1 / math.sqrt(128)))
    print(f"blocks a={a} s={s} window={window} zero_block={zb} {dtype}", flush=True)
    x = util.randn((a, s, s), dtype, seed=seed, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=seed + 1)
    eff = None if window is None or window >= s else window
    written = _written_blocks(s, zb, eff, "cpu")
    masked = fb.causal_mask(s, sliding_window_width=window)[0, 0]
    assert bool((written | masked).all())
    sentinel = 0x7e01
    want_y = oracle.causal_softmax_fwd(x, scale, window=window)
    want_dx = oracle.softmax_bwd(dy, want_y, scale, causal=True, window=window)
    real_empty = torch.empty_like

    def marked(t, **k):
        out = real_empty(t, **k)
        out.view(torch.int16).fill_(sentinel)
        return out

    def planted(t):
        t = t.clone()
        t.view(torch.int16)[:, ~written] = sentinel
        return t.to(DEV)

    torch.empty_like = marked
    try:
        y = ext.forward(x.to(DEV), scale, window, None, None, None, zb).cpu()
        dx = ext.backward(planted(dy), planted(want_y), scale, window, None, zb).cpu()
    finally:
        torch.empty_like = real_empty
    for got in (y, dx):
        if not bool(written.all()):
            assert bool((util.raw_bits(got)[:, ~written] == sentinel).all())
        zeros = written & masked
        assert int(util.raw_bits(got)[:, zeros].abs().max() if zeros.any() else 0) == 0
    util.assert_ulp_close(torch.where(written, y, want_y), want_y, 2, "y")
    util.assert_softmax_bwd_close(torch.where(written, dx, want_dx), want_dx, dy.masked_fill(masked, 0), want_y, scale, "dx")


@pytest.mark.parametrize("seed", [*range(20), 207])  # 207: an unmasked fp16 probability on the 0 / one-ulp rounding edge
def test_softmax_extras_with_dropout_random_shapes(hotpath, seed):
    """Both softmax kernels with a random subset of {AliBi, bias tensor, key lengths} and attention dropout, on
    shapes around the launch-geometry boundaries, through the extension modules: probabilities within 2 ulp of the
    oracle's composition, zeros (and uniform rows) where it has them, `dropped` exactly the oracle's dropout of the
    stored probabilities, the causal backward with key lengths against the oracle."""
    import scaled_masked_softmax_cuda as mext
    import scaled_upper_triang_masked_softmax_cuda as cext

    rng = random.Random(7000 + seed)
    dtype = rng.choice(HALF)
    b, heads = rng.randint(1, 3), rng.randint(1, 4)
    s = boundary_int(rng, 2, 1100)
    scale = rng.choice((1.0, 0.125, 1 / math.sqrt(128)))
    p, sd = rng.choice((0.1, 0.5)), rng.randint(0, 1 << 40)
    use = {k: rng.random() < 0.6 for k in "abl"}
    print(f"extras b={b} heads={heads} s={s} {dtype} use={use} p={p}", flush=True)
    slopes = torch.tensor(fb.alibi_slopes(max(heads, 2))[:heads], dtype=torch.float32) if use["a"] else None
    bias = util.randn((heads, s, s), dtype, seed=seed + 2, std=1.5) if use["b"] else None
    lengths = torch.tensor([rng.choice((0, s, rng.randint(0, s))) for _ in range(b)], dtype=torch.int32) if use["l"] else None
    x = util.randn((b, heads, s, s), dtype, seed=seed, std=2.0)
    dy = util.randn((b, heads, s, s), dtype, seed=seed + 1)
    dev = lambda t: None if t is None else t.to(DEV)

    # causal kernel
    want = oracle.causal_softmax_fwd(x.view(-1, s, s), scale, None, slopes, bias, lengths)
    dropped, y = [t.cpu() for t in cext.forward_dropout(x.view(-1, s, s).to(DEV), scale, p, sd, None, 0, dev(slopes), dev(bias),
                                                         dev(lengths))]
    util.assert_ulp_close(y, want, 2, "causal y")
    assert torch.equal(util.raw_bits(dropped), util.raw_bits(oracle.bias_dropout_add(y, None, None, p, sd)))
    want_dx = oracle.causal_softmax_dropout_bwd(dy.view(-1, s, s), want, scale, p, sd, key_lengths=lengths)
    got_dx = cext.backward_dropout(dy.view(-1, s, s).to(DEV).clone(), want.to(DEV), scale, p, sd, None, 0, dev(lengths)).cpu()
    g = oracle.bias_dropout_add(dy.view(-1, s, s), None, None, p, sd)
    keys = torch.arange(s)
    masked = fb.causal_mask(s)[0, 0].expand(b * heads, s, s).clone()
    if lengths is not None:
        masked |= (keys.view(1, 1, s) >= lengths.clamp(0, s).view(b, 1, 1)).repeat_interleave(heads, dim=0)
    # masked positions hold +0 exactly wherever the oracle has it (all but the uniform rows); an unmasked probability at the
    # edge of the subnormal range may round to 0 on one side and to one ulp on the other, which the 2-ulp bound covers
    assert not util.raw_bits(y)[masked & (util.raw_bits(want) == 0)].any()
    assert int(util.raw_bits(got_dx)[masked].abs().max() if masked.any() else 0) == 0
    util.assert_softmax_bwd_close(got_dx, want_dx, g.masked_fill(masked, 0), want, scale, "causal dx")

    # padding-mask kernel (sq > 1 is a precondition of the reference's entry point)
    if s > 1:
        mask = util.padding_mask(b, s, s, seed=seed, lo=1) | fb.causal_mask(s)
        if rng.random() < 0.5:
            mask = mask[:1].contiguous()
        want_m = oracle.masked_softmax_fwd(x, mask, scale, slopes, bias, lengths)
        dropped_m, y_m = [t.cpu() for t in mext.forward_dropout(x.to(DEV), mask.to(DEV), scale, p, sd, dev(slopes), dev(bias),
                                                                 dev(lengths))]
        util.assert_ulp_close(y_m, want_m, 2, "masked y")
        masked_m = mask.expand(b, heads, s, s).clone()
        if lengths is not None:
            masked_m |= (keys.view(1, 1, 1, s) >= lengths.clamp(0, s).view(b, 1, 1, 1)).expand_as(masked_m)
        masked_m &= util.raw_bits(want_m) == 0
        assert not util.raw_bits(y_m)[masked_m].any()
        assert torch.equal(util.raw_bits(dropped_m), util.raw_bits(oracle.bias_dropout_add(y_m, None, None, p, sd)))
        plain = mext.forward(x.to(DEV), mask.to(DEV), scale, dev(slopes), dev(bias), dev(lengths)).cpu()
        assert torch.equal(util.raw_bits(plain), util.raw_bits(y_m))
