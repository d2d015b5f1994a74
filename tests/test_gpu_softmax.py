"""GPU parity of the softmax kernels, called through the C ABI, against the CPU
oracle (oracle/kernel_semantics.c) on the same seeded inputs.

Tolerances (stated per assertion): forward probabilities within 2 ulp of the
storage dtype, masked positions bit-exact +0, fully masked rows exactly 1/sk;
backward within 2 ulp plus the fp32 row-sum rounding noise (util.assert_softmax_bwd_close).
"""
import math

import pytest
import torch

import oracle
import util

pytestmark = pytest.mark.gpu

DTYPES = [torch.bfloat16, torch.float16]
DEV = "cuda"


def say(*a):
    print(*a, flush=True)


# (attn_batches, seq_len): every register geometry of the chunked kernels
# (L=1..64, K=1..4, W=2,4), non-power-of-two lengths, row counts that do not
# fill a workgroup, and lengths that take the scalar kernel (s % 8 != 0).
CAUSAL_SHAPES = [
    (3, 8), (5, 16), (3, 24), (2, 40), (7, 64), (3, 128), (2, 200), (5, 256), (2, 264), (3, 512),
    (2, 1000), (2, 1024), (1, 1536), (2, 2048), (1, 2056), (1, 3072), (1, 4096), (1, 6144), (1, 8192),
    (3, 1), (3, 17), (2, 33), (1, 1001),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", CAUSAL_SHAPES, ids=lambda s: f"a{s[0]}_s{s[1]}")
def test_causal_forward_backward_vs_oracle(hotpath, shape, dtype):
    a, s = shape
    scale = 1.0 / math.sqrt(128.0)
    say(f"causal fwd/bwd a={a} s={s} {dtype}")
    x = util.randn((a, s, s), dtype, seed=s * 7 + a, std=2.0)
    dy = util.randn((a, s, s), dtype, seed=s * 11 + a)
    want_y = oracle.causal_softmax_fwd(x, scale)
    got_y = util.abi_causal_fwd(hotpath, x.to(DEV), scale)
    torch.cuda.synchronize()
    got_y_cpu = got_y.cpu()
    # masked positions: bit-exact +0
    upper = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
    assert int(util.raw_bits(got_y_cpu)[:, upper].abs().max() if upper.any() else 0) == 0
    # probabilities: within 2 ulp
    util.assert_ulp_close(got_y_cpu, want_y, 2, "causal fwd")
    # backward uses the oracle's y on both sides so that only the backward kernel is compared
    want_dx = oracle.softmax_bwd(dy, want_y, scale, causal=True)
    got_dx = util.abi_causal_bwd(hotpath, dy.to(DEV), want_y.to(DEV), scale)
    torch.cuda.synchronize()
    got_dx_cpu = got_dx.cpu()
    assert int(util.raw_bits(got_dx_cpu)[:, upper].abs().max() if upper.any() else 0) == 0
    util.assert_softmax_bwd_close(got_dx_cpu, want_dx, dy, want_y, scale, "causal bwd")
    # in-place call gives the same bits as the out-of-place one
    g = dy.to(DEV).clone()
    util.abi_causal_bwd(hotpath, g, want_y.to(DEV), scale, inplace=True)
    torch.cuda.synchronize()
    assert torch.equal(util.raw_bits(g.cpu()), util.raw_bits(got_dx_cpu))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("n,batches", [(512, 33), (504, 33), (256, 130), (136, 490), (64, 2050), (24, 21900), (8, 131100)],
                         ids=lambda v: str(v))
def test_causal_forward_short_rows_many_rows(hotpath, n, batches, dtype):
    """Rows of at most 512 keys in tensors with enough rows take a kernel of their own (four rows in flight per lane,
    the last workgroup ragged). Bit for bit the result of the same matrices handed over in groups small enough for
    the general kernel, which is the one the other tests compare with the oracle; a few matrices against the oracle
    here as well."""
    say(f"causal short rows n={n} batches={batches} {dtype}")
    x = util.randn((batches, n, n), dtype, seed=n, std=2.0).to(DEV)
    scale = 0.11
    got = util.abi_causal_fwd(hotpath, x, scale)
    step = max(1, (1 << 20) // (4 * n * max(8, n // 8)))  # far below the row count that selects the short-row kernel
    for b0 in list(range(0, batches, max(1, batches // 5)))[:5] + [batches - step]:
        part = util.abi_causal_fwd(hotpath, x[b0:b0 + step].contiguous(), scale)
        assert torch.equal(util.raw_bits(got[b0:b0 + step]), util.raw_bits(part)), b0
    for b0 in (0, batches - 1):
        want = oracle.causal_softmax_fwd(x[b0:b0 + 1].cpu(), scale)
        util.assert_ulp_close(got[b0:b0 + 1].cpu(), want, 2, f"matrix {b0}")
        assert (got[b0].cpu().float().triu(1) == 0).all()


@pytest.mark.parametrize("n,batches", [(512, 40), (136, 490), (24, 21900)], ids=lambda v: str(v))
@pytest.mark.parametrize("window", ["third", 0, "wide"])
def test_causal_forward_short_rows_many_rows_with_a_window(hotpath, n, batches, window):
    """The short-row kernel also serves a sliding window (nothing else: AliBi, bias, key lengths, dropout and block
    limits go to the general kernel). Bit for bit the general kernel's result on groups of matrices below the row
    count that selects the short-row kernel, and two matrices against the oracle."""
    w = {"third": n // 3, 0: 0, "wide": n + 5}[window]
    say(f"causal short rows with window n={n} batches={batches} window={w}")
    dtype = torch.bfloat16
    x = util.randn((batches, n, n), dtype, seed=n + 1, std=2.0).to(DEV)
    scale = 0.11

    def run(t):
        y = torch.empty_like(t)
        rc = hotpath.lib().nhp_causal_softmax_ex_fwd(y.data_ptr(), t.data_ptr(), scale, t.size(0), n, w, None, None, None, 1,
                                                     hotpath.BF16, None)
        assert rc == 0, hotpath.lib().nhp_status_string(rc)
        return y

    got = run(x)
    step = max(1, (1 << 20) // (4 * n * max(8, n // 8)))
    for b0 in list(range(0, batches, max(1, batches // 5)))[:5] + [batches - step]:
        part = run(x[b0:b0 + step].contiguous())
        assert torch.equal(util.raw_bits(got[b0:b0 + step]), util.raw_bits(part)), b0
    for b0 in (0, batches - 1):
        want = oracle.causal_softmax_fwd(x[b0:b0 + 1].cpu(), scale, window=w)
        util.assert_ulp_close(got[b0:b0 + 1].cpu(), want, 2, f"matrix {b0}")
        outside = ~fb_band(n, w)
        assert int(util.raw_bits(got[b0].cpu())[outside].abs().max()) == 0, "outside the band: +0 bit for bit"


def fb_band(n, w):
    q = torch.arange(n).view(n, 1)
    k = torch.arange(n).view(1, n)
    return (k <= q) & (k >= q - w)


def test_causal_forward_in_place(hotpath):
    x = util.randn((4, 512, 512), torch.bfloat16, seed=5, std=2.0).to(DEV)
    want = util.abi_causal_fwd(hotpath, x, 0.125)
    rc = hotpath.lib().nhp_causal_softmax_fwd(x.data_ptr(), x.data_ptr(), 0.125, 4, 512, hotpath.BF16, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(util.raw_bits(x.cpu()), util.raw_bits(want.cpu()))


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
def test_causal_closed_forms(hotpath, dtype):
    """Row q of a constant matrix is 1/(q+1) on k <= q; row 0 is [1, 0, ...]."""
    s = 1024
    x = torch.full((2, s, s), 3.0, dtype=dtype, device=DEV)
    y = util.abi_causal_fwd(hotpath, x, 0.3).cpu()
    q = torch.arange(s)
    want = torch.where(q[None, :] <= q[:, None], 1.0 / (q[:, None] + 1).float(), torch.zeros(())).to(dtype)
    assert torch.equal(util.raw_bits(y[0]), util.raw_bits(want))
    assert torch.equal(util.raw_bits(y[1]), util.raw_bits(want))
    assert y[0, 0, 0].item() == 1.0


def test_causal_wide_dynamic_range(hotpath):
    """Logit gaps up to ~100 (e^-100 ~ 3.7e-44): bf16 results down to the
    subnormal range must still match the oracle; nothing may turn into NaN."""
    s = 256
    g = torch.Generator().manual_seed(3)
    x = (torch.rand((2, s, s), generator=g) * 100.0).to(torch.bfloat16)
    want = oracle.causal_softmax_fwd(x, 1.0)
    got = util.abi_causal_fwd(hotpath, x.to(DEV), 1.0).cpu()
    assert not torch.isnan(got.float()).any()
    util.assert_ulp_close(got, want, 2, "wide range")


def test_causal_negative_and_zero_scale(hotpath):
    s = 128
    x = util.randn((2, s, s), torch.float16, seed=9, std=3.0)
    for scale in (-0.5, 0.0):
        want = oracle.causal_softmax_fwd(x, scale)
        got = util.abi_causal_fwd(hotpath, x.to(DEV), scale).cpu()
        util.assert_ulp_close(got, want, 2, f"scale {scale}")


# (b, np, sq, sk, pad_batches)
MASKED_SHAPES = [
    (2, 3, 4, 8, 2), (2, 2, 8, 32, 1), (3, 2, 6, 64, 3), (2, 4, 4, 128, 2), (2, 2, 12, 256, 1),
    (2, 3, 8, 512, 2), (2, 2, 4, 1000, 2), (2, 5, 4, 1024, 1), (1, 2, 4, 1536, 1), (2, 3, 8, 2048, 2),
    (1, 2, 4, 3000, 1), (2, 2, 4, 4096, 2), (1, 3, 2, 8192, 1), (1, 2, 2, 12288, 1), (1, 2, 2, 16384, 1),
    (1, 1, 2, 32768, 1), (1, 1, 2, 40960, 1), (1, 1, 2, 65536, 1),
    (2, 2, 4, 20, 2), (1, 2, 4, 1001, 1), (1, 1, 2, 65544, 1),
]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", MASKED_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_masked_forward_backward_vs_oracle(hotpath, shape, dtype):
    b, np_, sq, sk, pb = shape
    scale = 1.0 / math.sqrt(128.0)
    say(f"masked fwd/bwd {shape} {dtype}")
    x = util.randn((b, np_, sq, sk), dtype, seed=sk + b, std=3.0)
    # a few +-60 outliers, as in the padded-attention benchmark configuration
    g = torch.Generator().manual_seed(sk)
    hit = torch.rand(x.shape, generator=g) < 0.01
    sign = torch.where(torch.rand(x.shape, generator=g) < 0.5, -60.0, 60.0).to(dtype)
    x = torch.where(hit, sign, x)
    mask = util.padding_mask(pb, sq, sk, seed=sk * 3, full_batch=pb - 1 if pb > 1 else None)
    if pb == 1:
        mask[0, 0, 0, :] = True  # one fully masked row
    dy = util.randn((b, np_, sq, sk), dtype, seed=sk + 17)

    want_y = oracle.masked_softmax_fwd(x, mask, scale)
    got_y = util.abi_masked_fwd(hotpath, x.to(DEV), mask.to(DEV), scale)
    torch.cuda.synchronize()
    got_y_cpu = got_y.cpu()
    util.assert_ulp_close(got_y_cpu, want_y, 2, "masked fwd")
    # fully masked rows: exactly uniform (bit-identical to the oracle's 1/sk)
    mask_b = mask.expand(b, 1, sq, sk)
    full = mask_b.all(dim=-1).expand(b, np_, sq)
    if full.any():
        assert torch.equal(util.raw_bits(got_y_cpu)[full], util.raw_bits(want_y)[full])
        uniform = torch.tensor(1.0 / sk).to(dtype)
        assert torch.equal(got_y_cpu[full], uniform.expand_as(got_y_cpu[full]))
    # masked entries of partially masked rows: exact zeros
    part = mask_b.expand(b, np_, sq, sk) & ~full[..., None]
    assert int(util.raw_bits(got_y_cpu)[part].abs().max() if part.any() else 0) == 0

    want_dx = oracle.softmax_bwd(dy, want_y, scale, causal=False)
    got_dx = util.abi_masked_bwd(hotpath, dy.to(DEV), want_y.to(DEV), scale)
    torch.cuda.synchronize()
    util.assert_softmax_bwd_close(got_dx.cpu(), want_dx, dy, want_y, scale, "masked bwd")
    g2 = dy.to(DEV).clone()
    util.abi_masked_bwd(hotpath, g2, want_y.to(DEV), scale, inplace=True)
    torch.cuda.synchronize()
    assert torch.equal(util.raw_bits(g2.cpu()), util.raw_bits(got_dx.cpu()))


def test_masked_uint8_mask_values(hotpath):
    """Only the byte value 1 masks (scaled_masked_softmax.h:180): 0, 2, 255 do not."""
    b, np_, sq, sk = 1, 2, 4, 256
    x = util.randn((b, np_, sq, sk), torch.float16, seed=1, std=2.0)
    g = torch.Generator().manual_seed(2)
    mask = torch.randint(0, 4, (1, 1, sq, sk), generator=g).to(torch.uint8)
    mask[mask == 3] = 255
    want = oracle.masked_softmax_fwd(x, mask, 0.7)
    got = util.abi_masked_fwd(hotpath, x.to(DEV), mask.to(DEV), 0.7).cpu()
    util.assert_ulp_close(got, want, 2, "uint8 mask")
    assert (got[..., (mask == 2)[0, 0]].float() > 0).any()


def test_unaligned_pointers_take_scalar_kernel(hotpath):
    """A view that starts 2 bytes into an allocation is not 16-byte aligned."""
    s = 64
    buf = util.randn((2 * s * s + 1,), torch.bfloat16, seed=4, std=2.0)
    x = buf[1:].view(2, s, s)
    want = oracle.causal_softmax_fwd(x.clone(), 0.5)
    xd = buf.to(DEV)[1:].view(2, s, s)
    assert xd.data_ptr() % 16 != 0
    got = util.abi_causal_fwd(hotpath, xd, 0.5).cpu()
    util.assert_ulp_close(got, want, 2, "unaligned")


# ---------------------------------------------------------------------------
# full benchmark sizes: size-independent properties (no oracle run)
# ---------------------------------------------------------------------------
def _check_causal_properties(y, dtype):
    a, s, _ = y.shape
    # rows sum to 1 within n * 2^-9 (bf16) / 2^-12 (fp16) rounding of the terms
    sums = y.float().sum(-1)
    tol = 2.0**-8 if dtype == torch.bfloat16 else 2.0**-10
    assert (sums - 1).abs().max().item() < tol * 8
    # strictly upper triangle is +0 bit for bit: check through the integer view
    bits = y.view(torch.int16)
    rows = torch.randint(0, s - 1, (64,), device=y.device)
    for r in rows.tolist():
        assert int(bits[:, r, r + 1 :].abs().max()) == 0
    assert int(bits[:, 0, 1:].abs().max()) == 0
    assert (y[:, 0, 0] == 1).all()


def test_causal_full_size_properties_pythia_1p4b(hotpath):
    """[8*16, 2048, 2048] bf16: row sums, exact zeros, and agreement of a
    sampled slice with the oracle."""
    a, s = 128, 2048
    scale = 1.0 / math.sqrt(128.0)
    g = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn((a, s, s), generator=g, device=DEV) * 2).to(torch.bfloat16)
    y = util.abi_causal_fwd(hotpath, x, scale)
    torch.cuda.synchronize()
    _check_causal_properties(y, torch.bfloat16)
    for idx in (0, 77, 127):
        want = oracle.causal_softmax_fwd(x[idx : idx + 1].cpu(), scale)
        util.assert_ulp_close(y[idx : idx + 1].cpu(), want, 2, f"slice {idx}")
    dy = torch.randn((a, s, s), generator=g, device=DEV).to(torch.bfloat16)
    dx = util.abi_causal_bwd(hotpath, dy, y, scale)
    torch.cuda.synchronize()
    # gradient rows sum to ~0 (the softmax Jacobian annihilates constants)
    rs = dx.float().sum(-1).abs().max().item()
    assert rs < 0.05, rs
    for idx in (3, 100):
        want = oracle.softmax_bwd(dy[idx : idx + 1].cpu(), y[idx : idx + 1].cpu(), scale, causal=True)
        util.assert_softmax_bwd_close(dx[idx : idx + 1].cpu(), want, dy[idx : idx + 1].cpu(),
                                      y[idx : idx + 1].cpu(), scale, f"bwd slice {idx}")


def test_causal_long_rows_properties(hotpath):
    """s = 8192 (4 waves per row) at [4, 8192, 8192] and s = 16384 / 32768
    (8 / 16 waves per row) on one matrix: properties plus sampled rows."""
    scale = 1.0 / math.sqrt(128.0)
    for a, s in ((4, 8192), (1, 16384), (1, 32768)):
        say(f"long rows a={a} s={s}")
        g = torch.Generator(device=DEV).manual_seed(s)
        x = (torch.randn((a, s, s), generator=g, device=DEV) * 2).to(torch.bfloat16)
        y = util.abi_causal_fwd(hotpath, x, scale)
        torch.cuda.synchronize()
        _check_causal_properties(y, torch.bfloat16)
        # sampled rows against torch on the GPU in fp32 (library softmax)
        for r in (0, 1, 511, 512, 513, s // 2, s - 2, s - 1):
            ref = torch.softmax(x[0, r, : r + 1].float() * scale, -1).to(torch.bfloat16)
            util.assert_ulp_close(y[0, r, : r + 1].cpu(), ref.cpu(), 2, f"s={s} row {r}")
        del x, y
        torch.cuda.empty_cache()


def test_masked_full_size_properties(hotpath):
    """[16, 32, 1024, 2048] fp16 with per-sequence valid lengths and one fully
    masked sequence: sampled (b, h) slices against the oracle, row sums."""
    b, np_, sq, sk = 16, 32, 1024, 2048
    scale = 1.0 / math.sqrt(128.0)
    g = torch.Generator(device=DEV).manual_seed(0)
    x = (torch.randn((b, np_, sq, sk), generator=g, device=DEV) * 3).to(torch.float16)
    hit = torch.rand(x.shape, generator=g, device=DEV) < 0.01
    x = torch.where(hit, torch.where(torch.rand(x.shape, generator=g, device=DEV) < 0.5, -60.0, 60.0).half(), x)
    del hit
    mask = util.padding_mask(b, sq, sk, seed=0, full_batch=7, lo=512).to(DEV)
    y = util.abi_masked_fwd(hotpath, x, mask, scale)
    torch.cuda.synchronize()
    sums = y.float().sum(-1)
    assert (sums - 1).abs().max().item() < 2e-2
    assert (y[7] == torch.tensor(1.0 / sk, dtype=torch.float16)).all()
    for bi, h in ((0, 0), (7, 5), (15, 31), (3, 16)):
        want = oracle.masked_softmax_fwd(x[bi : bi + 1, h : h + 1, :64].cpu(), mask[bi : bi + 1, :, :64].cpu(), scale)
        util.assert_ulp_close(y[bi : bi + 1, h : h + 1, :64].cpu(), want, 2, f"slice {bi},{h}")
    dy = torch.randn(x.shape, generator=g, device=DEV).half()
    del x
    dx = util.abi_masked_bwd(hotpath, dy, y, scale)
    torch.cuda.synchronize()
    for bi, h in ((0, 0), (7, 5), (15, 31)):
        sl = (slice(bi, bi + 1), slice(h, h + 1), slice(0, 64))
        want = oracle.softmax_bwd(dy[sl].cpu(), y[sl].cpu(), scale, causal=False)
        util.assert_softmax_bwd_close(dx[sl].cpu(), want, dy[sl].cpu(), y[sl].cpu(), scale, f"bwd {bi},{h}")


def test_causal_llama2_7b_full_size_64bit_indexing(hotpath):
    """[2*32, 8192, 8192] bf16 = 2^32 elements per tensor (8 GiB): element offsets
    exceed 32 bits. Properties over the whole tensor, and the last matrices (beyond
    2^31 elements) against torch on the GPU and the oracle on sampled rows."""
    a, s = 64, 8192
    scale = 1.0 / math.sqrt(128.0)
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.empty((a, s, s), dtype=torch.bfloat16, device=DEV)
    for i in range(0, a, 8):  # generate in slices to bound the fp32 temporaries
        x[i : i + 8] = (torch.randn((8, s, s), generator=g, device=DEV) * 2).to(torch.bfloat16)
    say("c5 forward")
    y = util.abi_causal_fwd(hotpath, x, scale)
    torch.cuda.synchronize()
    for m in (0, 31, 32, 63):
        sums = y[m].float().sum(-1)
        assert (sums - 1).abs().max().item() < 0.05
        assert int(y[m].view(torch.int16).triu(1).abs().max()) == 0
        for r in (0, 511, 512, 4095, 8191):
            ref = torch.softmax(x[m, r, : r + 1].float() * scale, -1).to(torch.bfloat16)
            util.assert_ulp_close(y[m, r, : r + 1].cpu(), ref.cpu(), 2, f"matrix {m} row {r}")
    rows = slice(8000, 8016)
    want = oracle.causal_softmax_fwd(x[63:64].cpu(), scale)[0, rows]
    util.assert_ulp_close(y[63, rows].cpu(), want, 2, "oracle rows of the last matrix")
    say("c5 backward")
    dy = torch.empty_like(x)
    for i in range(0, a, 8):
        dy[i : i + 8] = torch.randn((8, s, s), generator=g, device=DEV).to(torch.bfloat16)
    keep = dy[63, rows].cpu()
    dx = util.abi_causal_bwd(hotpath, dy, y, scale, inplace=True)
    torch.cuda.synchronize()
    for m in (0, 32, 63):
        assert int(dx[m].view(torch.int16).triu(1).abs().max()) == 0
        assert dx[m].float().sum(-1).abs().max().item() < 0.05
    # rows 8000..8015 of the last matrix against the oracle (the oracle wants whole matrices: build one
    # whose other rows are zero, which leaves these rows unchanged)
    yc = torch.zeros((1, s, s), dtype=torch.bfloat16)
    gc = torch.zeros((1, s, s), dtype=torch.bfloat16)
    yc[0, rows] = y[63, rows].cpu()
    gc[0, rows] = keep
    want_dx = oracle.softmax_bwd(gc, yc, scale, causal=True)[0, rows]
    util.assert_softmax_bwd_close(dx[63, rows].cpu(), want_dx, gc[0, rows], yc[0, rows], scale, "bwd rows of the last matrix")


def test_empty_tensors_through_the_modules():
    import scaled_masked_softmax_cuda as masked
    import scaled_upper_triang_masked_softmax_cuda as causal

    e = torch.empty((0, 64, 64), dtype=torch.bfloat16, device=DEV)
    assert causal.forward(e, 1.0).shape == (0, 64, 64)
    assert causal.backward(e.clone(), e, 1.0).shape == (0, 64, 64)
    e4 = torch.empty((0, 4, 8, 64), dtype=torch.float16, device=DEV)
    m4 = torch.empty((0, 1, 8, 64), dtype=torch.bool, device=DEV)
    assert masked.forward(e4, m4, 1.0).shape == (0, 4, 8, 64)
    assert masked.backward(e4.clone(), e4, 1.0).shape == (0, 4, 8, 64)


def test_hip_graph_capture_and_replay(hotpath):
    """The library allocates nothing and never synchronises, so its launches can be
    captured in a HIP graph. Every replay (with eager work and synchronisation in
    between) must give the eager result bit for bit."""
    a, s, scale = 16, 1024, 0.125
    x = util.randn((a, s, s), torch.bfloat16, seed=1, std=2.0).to(DEV)
    dy = util.randn((a, s, s), torch.bfloat16, seed=2).to(DEV)
    y = torch.empty_like(x)
    dx = torch.empty_like(x)
    L = hotpath.lib()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream
        L.nhp_causal_softmax_fwd(y.data_ptr(), x.data_ptr(), scale, a, s, hotpath.BF16, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = torch.cuda.current_stream().cuda_stream
        assert L.nhp_causal_softmax_fwd(y.data_ptr(), x.data_ptr(), scale, a, s, hotpath.BF16, st) == 0
        assert L.nhp_causal_softmax_bwd(dx.data_ptr(), dy.data_ptr(), y.data_ptr(), scale, a, s, hotpath.BF16, st) == 0
    for rep in range(3):
        x.copy_(util.randn((a, s, s), torch.bfloat16, seed=10 + rep, std=2.0).to(DEV))
        y.fill_(7)
        dx.fill_(7)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want_y = util.abi_causal_fwd(hotpath, x, scale)
        want_dx = util.abi_causal_bwd(hotpath, dy, want_y, scale)
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), want_y.view(torch.int16)), rep
        assert torch.equal(dx.view(torch.int16), want_dx.view(torch.int16)), rep
