"""GPU parity of the rotary kernels, called through the C ABI, against the CPU
oracle and against eager torch.

Cached tables: bit-exact (the kernel performs the same three roundings as the
scalar types of the reference). On-device cos/sin (freqs variant): the fp32
sincos of the device and of the host libm may differ in the last places, which
can only change a table entry whose exact value lies next to a rounding
boundary of the data dtype. Those entries are located on the host; every
element that does not depend on one must be bit-identical to the oracle, the
others (a fraction of a per cent, asserted) within two spacings at the
magnitude of the inputs (util.assert_rope_freqs_close).
"""
import pytest
import torch

import oracle
import util
from oracle import fallback_semantics as fb

pytestmark = pytest.mark.gpu
DEV = "cuda"


def say(*a):
    print(*a, flush=True)


def tables(d2, s, dtype, cs_fp32=False):
    """Tables of the RotaryEmbedding recipe (the two halves of the feature axis share angles)."""
    cos, sin, ang = fb.rotary_tables(d2, s, 10000, torch.float32 if cs_fp32 else dtype)
    return cos.contiguous(), sin.contiguous(), ang.contiguous()


def generic_tables(d2, s, dtype, cs_fp32=False, seed=0):
    """Independent angle for every (position, feature): unlike the recipe above this tells
    sin[i] from sin[i + d2/2], and it exists for odd d2."""
    g = torch.Generator().manual_seed(seed)
    ang = (torch.rand((s, 1, 1, d2), generator=g) * 20.0 - 10.0).contiguous()
    cs = torch.float32 if cs_fp32 else dtype
    return ang.cos().to(cs).contiguous(), ang.sin().to(cs).contiguous(), ang


# (s, b, h, d, d2)
SHAPES = [
    (16, 2, 4, 128, 128), (16, 2, 4, 128, 32), (9, 3, 5, 64, 64), (8, 2, 3, 96, 96), (8, 2, 3, 80, 48),
    (5, 2, 33, 128, 64), (4, 1, 2, 256, 256), (7, 2, 2, 32, 16), (3, 2, 2, 24, 8), (6, 2, 3, 20, 10),
    (4, 2, 2, 16, 6), (4, 2, 2, 15, 7), (64, 4, 16, 128, 32), (33, 5, 40, 128, 128),
]
# rotary dimensions whose half is not a whole number of 16-byte chunks (a quarter of the head sizes 96 and 80, the
# rotary slice passed on its own, an odd half) take the gather kernel; several row steps per workgroup, ragged rows
GATHER_SHAPES = [(33, 2, 5, 96, 24), (17, 3, 4, 80, 20), (16, 2, 3, 24, 24), (12, 1, 7, 512, 40), (5, 3, 47, 96, 24),
                 (9, 2, 2, 48, 6), (6, 2, 70, 32, 12)]
SHAPES = SHAPES + GATHER_SHAPES
DTYPES = [torch.bfloat16, torch.float16, torch.float32]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("cs_fp32", [False, True], ids=["cs_same", "cs_fp32"])
def test_rope_cached_bit_exact(hotpath, shape, dtype, cs_fp32):
    s, b, h, d, d2 = shape
    say(f"rope cached {shape} {dtype} cs_fp32={cs_fp32}")
    t = util.randn((s, b, h, d), dtype, seed=s + d)
    cos, sin, _ = generic_tables(d2, s, dtype, cs_fp32, seed=d2)
    for backward in (False, True):
        for transpose in (False, True):
            want = oracle.rope_cached(t, cos, sin, backward=backward, transpose_output=transpose)
            got = util.abi_rope_cached(hotpath, t.to(DEV), cos.to(DEV), sin.to(DEV), backward, transpose)
            torch.cuda.synchronize()
            assert got.stride() == want.stride()
            assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(want)), (backward, transpose)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
def test_rope_strided_views_of_fused_qkv(hotpath, dtype):
    """q, k as NeoX passes them: slices of a [sq, b, np, 3*hn] projection, and
    the partial-rotary narrowing [..., :rot] on top (transformer.py:852-887)."""
    s, b, h, hn = 32, 2, 8, 128
    qkv = util.randn((s, b, h, 3 * hn), dtype, seed=1)
    qkv_d = qkv.to(DEV)
    for d2 in (128, 32):
        cos, sin, _ = tables(d2, s, dtype)
        for part in range(2):
            view = qkv[..., part * hn : (part + 1) * hn]
            view_d = qkv_d[..., part * hn : (part + 1) * hn]
            for backward in (False, True):
                # full head vector with in-kernel pass-through
                want = oracle.rope_cached(view, cos, sin, backward=backward)
                got = util.abi_rope_cached(hotpath, view_d, cos.to(DEV), sin.to(DEV), backward)
                assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(want))
                # narrowed view, d == d2
                want = oracle.rope_cached(view[..., :d2], cos, sin, backward=backward)
                got = util.abi_rope_cached(hotpath, view_d[..., :d2], cos.to(DEV), sin.to(DEV), backward)
                assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(want))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "fp16", "fp32"])
def test_rope_matches_eager_torch(hotpath, dtype):
    """Forward equals apply_rotary_pos_emb_torch bit for bit; backward equals
    autograd through the eager expression when that is evaluated with the same
    roundings (the adjoint rotation)."""
    s, b, h, d = 24, 2, 4, 128
    for d2 in (128, 32):
        t = util.randn((s, b, h, d), dtype, seed=d2)
        cos, sin, _ = tables(d2, s, dtype)
        want = fb.eager_rotary_partial(t, cos, sin)
        got = util.abi_rope_cached(hotpath, t.to(DEV), cos.to(DEV), sin.to(DEV)).cpu()
        assert torch.equal(util.raw_bits(got), util.raw_bits(want))
        # backward: rotation by the negative angle = forward with sin -> -sin
        g = util.randn((s, b, h, d), dtype, seed=d2 + 1)
        want_b = fb.eager_rotary_partial(g, cos, -sin)
        got_b = util.abi_rope_cached(hotpath, g.to(DEV), cos.to(DEV), sin.to(DEV), backward=True).cpu()
        assert torch.equal(util.raw_bits(got_b), util.raw_bits(want_b))


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", SHAPES[:8] + SHAPES[12:14] + GATHER_SHAPES[:3], ids=lambda s: "x".join(map(str, s)))
def test_rope_freqs_vs_oracle(hotpath, shape, dtype):
    s, b, h, d, d2 = shape
    say(f"rope freqs {shape} {dtype}")
    t = util.randn((s, b, h, d), dtype, seed=s + d + 1)
    _, _, ang = generic_tables(d2, s, dtype, seed=d)
    # include large angles (positions in the thousands) to exercise range reduction
    ang = (ang * torch.where(torch.arange(s) % 2 == 0, 1.0, 700.0).view(s, 1, 1, 1)).contiguous()
    for backward in (False, True):
        want = oracle.rope_freqs(t, ang, backward=backward)
        got = util.abi_rope_freqs(hotpath, t.to(DEV), ang.to(DEV), backward)
        torch.cuda.synchronize()
        share = util.assert_rope_freqs_close(got, want, t, ang, backward, f"rope freqs {shape} {dtype} bwd={backward}")
        say(f"  share of elements on a table rounding boundary: {share:.5f}")
        # pass-through features are copies
        if d > d2:
            assert torch.equal(util.raw_bits(got.cpu()[..., d2:]), util.raw_bits(t[..., d2:]))


def test_rope_full_size_properties(hotpath):
    """q, k [4096, 4, 32, 128] bf16 (rotary_pct 1.0 and 0.25) and the
    Llama-2-7B shape [8192, 2, 32, 128]: bit-exact against eager torch on the
    GPU (same roundings), position 0 is the identity, tail features are copies,
    and backward(forward(x)) returns x up to the six roundings involved."""
    for (s, b, h, d), pcts in (((4096, 4, 32, 128), (1.0, 0.25)), ((8192, 2, 32, 128), (1.0,))):
        for pct in pcts:
            d2 = int(d * pct)
            say(f"rope full size s={s} b={b} h={h} d={d} d2={d2}")
            g = torch.Generator(device=DEV).manual_seed(s + d2)
            q = torch.randn((s, b, h, d), generator=g, device=DEV).to(torch.bfloat16)
            cos, sin, _ = tables(d2, s, torch.bfloat16)
            cos, sin = cos.to(DEV), sin.to(DEV)
            y = util.abi_rope_cached(hotpath, q, cos, sin)
            want = fb.eager_rotary_partial(q, cos, sin)
            assert torch.equal(y.view(torch.int16), want.view(torch.int16))
            assert torch.equal(y[0].view(torch.int16), q[0].view(torch.int16))
            if d2 < d:
                assert torch.equal(y[..., d2:].contiguous().view(torch.int16), q[..., d2:].contiguous().view(torch.int16))
            back = util.abi_rope_cached(hotpath, y, cos, sin, backward=True)
            err = (back.float() - q.float()).abs().max().item()
            assert err < 0.1, err
            # adjointness <rope(x), g> == <x, rope_bwd(g)> up to bf16 rounding
            gy = torch.randn((s, b, h, d), generator=g, device=DEV).to(torch.bfloat16)
            gx = util.abi_rope_cached(hotpath, gy, cos, sin, backward=True)
            lhs = (y.double() * gy.double()).sum().item()
            rhs = (q.double() * gx.double()).sum().item()
            # each of the ~N products carries a relative rounding error of about 2^-8 with random
            # sign, so the two sums differ by a few times 2^-8 * sqrt(sum of squared terms);
            # a wrong sign or index in backward would move rhs by about sqrt(N) instead
            noise = 2.0**-8 * (y.double() * gy.double()).pow(2).sum().item() ** 0.5
            assert abs(lhs - rhs) <= 8 * noise, (lhs, rhs, noise)


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(16, 2, 8, 8, 128, 128), (16, 2, 8, 2, 128, 32), (9, 3, 5, 1, 64, 16), (7, 2, 4, 4, 24, 8),
                                   (11, 2, 6, 2, 96, 24)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rope_qk_single_launch_equals_two_calls(hotpath, shape, dtype):
    """q and k (k possibly with fewer heads) through nhp_rope_cached_qk_* give the
    bits of two nhp_rope_cached_* calls, forward and backward, for views of a
    fused projection and for both output layouts."""
    s, b, hq, hk, d, d2 = shape
    buf = util.randn((s, b, hq + 2 * hk, d), dtype, seed=s + d).to(DEV)
    q, k = buf[:, :, :hq], buf[:, :, hq : hq + hk]
    cos, sin, _ = generic_tables(d2, s, dtype, seed=d2)
    cos, sin = cos.to(DEV), sin.to(DEV)
    L = hotpath.lib()
    for backward in (False, True):
        for transpose in (False, True):
            want_q = util.abi_rope_cached(hotpath, q, cos, sin, backward, transpose)
            want_k = util.abi_rope_cached(hotpath, k, cos, sin, backward, transpose)
            got_q = util._rope_out(q, transpose)
            got_k = util._rope_out(k, transpose)
            fn = L.nhp_rope_cached_qk_bwd if backward else L.nhp_rope_cached_qk_fwd
            rc = fn(got_q.data_ptr(), got_k.data_ptr(), q.data_ptr(), k.data_ptr(), cos.data_ptr(), sin.data_ptr(), s, b,
                    hq, hk, d, d2, hotpath.strides4(q), hotpath.strides4(k), hotpath.strides4(got_q),
                    hotpath.strides4(got_k), hotpath.dtype_code(q, "t"), hotpath.dtype_code(cos, "c"), None)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(util.raw_bits(got_q.cpu()), util.raw_bits(want_q.cpu()))
            assert torch.equal(util.raw_bits(got_k.cpu()), util.raw_bits(want_k.cpu()))
            # and against the oracle directly
            assert torch.equal(util.raw_bits(got_k.cpu()), util.raw_bits(oracle.rope_cached(k.cpu(), cos.cpu(), sin.cpu(), backward, transpose)))


@pytest.mark.parametrize("d,d2", [(16, 16), (32, 8), (24, 12), (16, 6), (8, 8), (32, 0)], ids=lambda v: str(v))
def test_rope_more_positions_than_a_grid_dimension_and_no_rotary_part(hotpath, d, d2):
    """The two-rows-per-thread kernel keeps the position in a grid dimension (at most 65535) and needs a rotary
    part; longer sequences, head vectors of a single chunk and d2 = 0 take the looping vector kernels (or, for
    a rotary half that is not a whole number of chunks, their gathering variant). Bit-exact like the others."""
    dtype = torch.bfloat16
    s, b, h = (65536 + 40, 1, 3) if d2 else (40, 2, 3)
    t = util.randn((s, b, h, d), dtype, seed=d + d2)
    cos, sin, _ = generic_tables(max(d2, 2), s, dtype, seed=d2)
    cos, sin = cos[..., :d2].contiguous(), sin[..., :d2].contiguous()
    td, cos_d, sin_d = t.to(DEV), cos.to(DEV), sin.to(DEV)
    for backward in (False, True):
        out = util._rope_out(td, False)
        fn = hotpath.lib().nhp_rope_cached_bwd if backward else hotpath.lib().nhp_rope_cached_fwd
        rc = fn(out.data_ptr(), td.data_ptr(), cos_d.data_ptr(), sin_d.data_ptr(), s, b, h, d, d2,
                hotpath.strides4(td), hotpath.strides4(out), hotpath.BF16, hotpath.BF16, None)
        assert rc == 0, hotpath.lib().nhp_status_string(rc)
        torch.cuda.synchronize()
        if d2:
            want = oracle.rope_cached(t, cos, sin, backward)
        else:
            want = t
        assert torch.equal(util.raw_bits(out.cpu()), util.raw_bits(want)), backward


# (s, b, h, d, d2): head vectors of 2..64 chunks, rows that do not fill the last workgroup, partial rotary dimensions
FUSED_QKV = [(16, 2, 8, 128, 128), (16, 2, 8, 128, 32), (5, 3, 7, 64, 64), (9, 1, 3, 32, 16), (3, 2, 5, 16, 16),
             (4, 2, 3, 256, 64), (3, 1, 2, 512, 512), (6, 2, 33, 128, 64), (64, 4, 16, 128, 128)]


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", FUSED_QKV, ids=lambda s: "x".join(map(str, s)))
def test_rope_qk_sliced_from_a_fused_projection(hotpath, shape, dtype):
    """q and k the way the attention layer slices them (megatron/model/transformer.py:852-866): last-dimension
    slices [..., :d] and [..., d:2d] of one [s, b, h, 3d] buffer, so k's head vector lies directly behind q's.
    The two-tensor entry points then read each (q|k) pair as one run; results are the oracle's bit for bit, in
    both directions and output layouts, with cached tables and with angles. Slices in another order, or with
    unequal strides, take the ordinary two-tensor launch and give the same bits."""
    s, b, h, d, d2 = shape
    say(f"rope q,k sliced from a fused buffer {shape} {dtype}")
    buf = util.randn((s, b, h, 3 * d), dtype, seed=s + d + d2).to(DEV)
    q, k, v = buf[..., :d], buf[..., d:2 * d], buf[..., 2 * d:]
    assert k.data_ptr() == q.data_ptr() + d * buf.element_size() and q.stride() == k.stride()
    cos, sin, ang = generic_tables(d2, s, dtype, seed=d2)
    cos_d, sin_d, ang_d = cos.to(DEV), sin.to(DEV), ang.to(DEV)
    L = hotpath.lib()
    code = hotpath.dtype_code(q, "t")
    for backward in (False, True):
        for transpose in (False, True):
            want_q = oracle.rope_cached(q.cpu(), cos, sin, backward, transpose)
            want_k = oracle.rope_cached(k.cpu(), cos, sin, backward, transpose)
            for first, second, want_first, want_second in ((q, k, want_q, want_k), (k, q, want_k, want_q), (k, v, want_k, None)):
                got_a, got_b = util._rope_out(first, transpose), util._rope_out(second, transpose)
                fn = L.nhp_rope_cached_qk_bwd if backward else L.nhp_rope_cached_qk_fwd
                rc = fn(got_a.data_ptr(), got_b.data_ptr(), first.data_ptr(), second.data_ptr(), cos_d.data_ptr(),
                        sin_d.data_ptr(), s, b, h, h, d, d2, hotpath.strides4(first), hotpath.strides4(second),
                        hotpath.strides4(got_a), hotpath.strides4(got_b), code, code, None)
                assert rc == 0, L.nhp_status_string(rc)
                torch.cuda.synchronize()
                assert torch.equal(util.raw_bits(got_a.cpu()), util.raw_bits(want_first)), (backward, transpose)
                if want_second is not None:
                    assert torch.equal(util.raw_bits(got_b.cpu()), util.raw_bits(want_second)), (backward, transpose)
            # the angles variant: the same bits as its single-tensor entry point (same device sine and cosine)
            got_a, got_b = util._rope_out(q, transpose), util._rope_out(k, transpose)
            fn = L.nhp_rope_freqs_qk_bwd if backward else L.nhp_rope_freqs_qk_fwd
            rc = fn(got_a.data_ptr(), got_b.data_ptr(), q.data_ptr(), k.data_ptr(), ang_d.data_ptr(), s, b, h, h, d, d2,
                    hotpath.strides4(q), hotpath.strides4(k), hotpath.strides4(got_a), hotpath.strides4(got_b), code, None)
            assert rc == 0, L.nhp_status_string(rc)
            torch.cuda.synchronize()
            assert torch.equal(util.raw_bits(got_a.cpu()),
                               util.raw_bits(util.abi_rope_freqs(hotpath, q, ang_d, backward, transpose).cpu()))
            assert torch.equal(util.raw_bits(got_b.cpu()),
                               util.raw_bits(util.abi_rope_freqs(hotpath, k, ang_d, backward, transpose).cpu()))
    # the buffer itself is untouched, v included
    assert torch.equal(util.raw_bits(buf.cpu()), util.raw_bits(util.randn((s, b, h, 3 * d), dtype, seed=s + d + d2)))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("offset", [0, 5])
def test_fused_qk_function_matches_eager_apply_with_offset(dtype, offset):
    """fused_apply_rotary_pos_emb_qk_cached == apply_rotary_pos_emb_torch on the rotary
    slice + concatenation of the pass-through slice (what ParallelSelfAttention does),
    including a position offset, forward and backward."""
    from megatron.model.fused_rope import fused_apply_rotary_pos_emb_qk_cached
    from megatron.model.positional_embeddings import RotaryEmbedding, apply_rotary_pos_emb_torch

    sq, b, hq, hk, d, d2, smax = 24, 2, 8, 2, 128, 32, 64
    rot = RotaryEmbedding(d2, smax, precision=dtype)
    q = util.randn((sq, b, hq, d), dtype, seed=1)
    k = util.randn((sq, b, hk, d), dtype, seed=2)
    gq = util.randn((sq, b, hq, d), dtype, seed=3)
    gk = util.randn((sq, b, hk, d), dtype, seed=4)
    # eager reference on the CPU: rotate the first d2 features, pass the rest through
    qe = q.clone().requires_grad_(True)
    ke = k.clone().requires_grad_(True)
    cos_c, sin_c = rot.cos_cached, rot.sin_cached
    oq = torch.cat((fb.eager_rotary(qe[..., :d2], cos_c, sin_c, offset), qe[..., d2:]), dim=-1)
    ok = torch.cat((fb.eager_rotary(ke[..., :d2], cos_c, sin_c, offset), ke[..., d2:]), dim=-1)
    torch.autograd.backward([oq, ok], [gq, gk])
    # and the two-operand eager function of the module agrees with that on the rotary slice
    eq, ek = apply_rotary_pos_emb_torch(q[..., :d2], k[..., :d2], cos_c, sin_c, offset)
    assert torch.equal(util.raw_bits(eq), util.raw_bits(oq[..., :d2].detach().contiguous()))
    qd = q.to(DEV).requires_grad_(True)
    kd = k.to(DEV).requires_grad_(True)
    cos, sin = rot(qd, seq_len=smax)
    fq, fk = fused_apply_rotary_pos_emb_qk_cached(qd, kd, cos, sin, offset)
    torch.autograd.backward([fq, fk], [gq.to(DEV), gk.to(DEV)])
    assert torch.equal(util.raw_bits(fq.detach().cpu()), util.raw_bits(oq.detach()))
    assert torch.equal(util.raw_bits(fk.detach().cpu()), util.raw_bits(ok.detach()))
    assert torch.equal(util.raw_bits(qd.grad.cpu()), util.raw_bits(qe.grad))
    assert torch.equal(util.raw_bits(kd.grad.cpu()), util.raw_bits(ke.grad))


# (s, b, h, d, d2): tile boundaries (s around 64), every number of load passes, partial rotary, shapes the
# transposing kernel refuses (s not a multiple of 8, d beyond 256) and that fall back to the scalar kernel
SEQ_MAJOR = [(64, 2, 3, 128, 128), (200, 2, 4, 128, 32), (72, 1, 5, 64, 64), (136, 2, 2, 96, 48), (8, 2, 2, 80, 16),
             (256, 1, 2, 256, 256), (120, 3, 2, 128, 64), (30, 2, 2, 128, 32), (16, 1, 2, 512, 64),
             # half the rotary dimension is not a whole number of chunks: rotated element by element
             (72, 2, 3, 96, 24), (136, 1, 4, 80, 20), (64, 2, 2, 64, 8), (40, 1, 3, 96, 96 - 8), (200, 2, 2, 128, 6)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", SEQ_MAJOR, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("cs_fp32", [False, True], ids=["cs_same", "cs_fp32"])
def test_rope_input_contiguous_along_the_sequence(hotpath, shape, dtype, cs_fp32):
    """The layout in which the key gradient reaches the rotary backward in the attention layer: the backward of
    the score GEMM leaves it as [b, h, d, s], seen as [s, b, h, d] with element strides (1, h*d*s, d*s, s)
    (megatron/model/transformer.py:556-562 and autograd's baddbmm formula). Bit-exact like every other layout."""
    s, b, h, d, d2 = shape
    say(f"rope sequence-major {shape} {dtype} cs_fp32={cs_fp32}")
    base = util.randn((b, h, d, s), dtype, seed=s + d)
    t = base.permute(3, 0, 1, 2)
    t_d = base.to(DEV).permute(3, 0, 1, 2)
    assert t_d.stride() == (1, h * d * s, d * s, s)
    cos, sin, _ = generic_tables(d2, s, dtype, cs_fp32, seed=d2)
    for backward in (False, True):
        for transpose in (False, True):
            want = oracle.rope_cached(t.contiguous(), cos, sin, backward=backward, transpose_output=transpose)
            got = util.abi_rope_cached(hotpath, t_d, cos.to(DEV), sin.to(DEV), backward, transpose)
            assert got.stride() == want.stride()
            assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(want)), (backward, transpose)
    # a window of a longer sequence: the feature stride exceeds the number of positions
    if s >= 16:
        w = t_d[8:s - 0]
        want = oracle.rope_cached(t[8:].contiguous(), cos[: s - 8].contiguous(), sin[: s - 8].contiguous(), backward=True)
        got = util.abi_rope_cached(hotpath, w, cos[: s - 8].contiguous().to(DEV), sin[: s - 8].contiguous().to(DEV), True)
        assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(want))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(64, 2, 3, 128, 128), (200, 2, 4, 128, 32), (136, 2, 2, 96, 48), (256, 1, 2, 256, 256),
                                   (72, 2, 3, 96, 24), (136, 1, 4, 80, 20)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rope_from_angles_on_input_contiguous_along_the_sequence(hotpath, shape, dtype):
    """The angles variant on the sequence-major layout takes the transposing kernel as well: same results as on
    the contiguous copy of the input bit for bit, and the oracle's to the tolerance of the angles variant."""
    s, b, h, d, d2 = shape
    say(f"rope freqs sequence-major {shape} {dtype}")
    base = util.randn((b, h, d, s), dtype, seed=s + d + 1)
    t = base.permute(3, 0, 1, 2)
    t_d = base.to(DEV).permute(3, 0, 1, 2)
    ang = (util.randn((s, 1, 1, d2), torch.float32, seed=d2 + 5) * 3.0).contiguous()
    for backward in (False, True):
        got = util.abi_rope_freqs(hotpath, t_d, ang.to(DEV), backward)
        same = util.abi_rope_freqs(hotpath, t_d.contiguous(), ang.to(DEV), backward)
        assert torch.equal(util.raw_bits(got.cpu()), util.raw_bits(same.cpu())), backward
        want = oracle.rope_freqs(t.contiguous(), ang, backward=backward)
        util.assert_rope_freqs_close(got.cpu(), want, t.contiguous(), ang, backward, f"seq-major freqs bwd={backward}")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "fp16"])
@pytest.mark.parametrize("shape", [(200, 10, 103, 64, 32), (72, 3, 1367, 64, 64), (2048, 2, 16, 128, 32), (136, 5, 99, 96, 24)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rope_from_angles_sequence_major_many_rows(hotpath, shape, dtype):
    """With many (batch, head) rows a workgroup of the transposing kernel evaluates the sines and cosines of its
    64 positions once and serves several rows with them (4, 8 and 1 rows per workgroup for these shapes, the
    last group ragged): bit for bit the result of the contiguous layout, which takes the other vector kernel."""
    s, b, h, d, d2 = shape
    say(f"rope freqs sequence-major, many rows {shape} {dtype}")
    t_d = util.randn((b, h, d, s), dtype, seed=s + h).to(DEV).permute(3, 0, 1, 2)
    ang = (util.randn((s, 1, 1, d2), torch.float32, seed=d2 + 6) * 3.0).contiguous().to(DEV)
    for backward in (False, True):
        got = util.abi_rope_freqs(hotpath, t_d, ang, backward)
        same = util.abi_rope_freqs(hotpath, t_d.contiguous(), ang, backward)
        assert torch.equal(util.raw_bits(got), util.raw_bits(same)), backward


@pytest.mark.parametrize("dtype", DTYPES, ids=["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("shape", [(16, 2, 8, 8, 128, 128), (16, 2, 8, 2, 128, 32), (9, 3, 5, 1, 64, 16), (7, 2, 4, 4, 24, 8),
                                   (11, 2, 6, 2, 96, 24)],
                         ids=lambda s: "x".join(map(str, s)))
def test_rope_from_angles_qk_single_launch_equals_two_calls(hotpath, shape, dtype):
    """nhp_rope_freqs_qk_* against two nhp_rope_freqs_* calls bit for bit (same device sine and cosine), forward and
    backward, on views of a fused projection, and through the autograd function against the per-tensor function."""
    from megatron.model.fused_rope import fused_apply_rotary_pos_emb, fused_apply_rotary_pos_emb_qk

    s, b, hq, hk, d, d2 = shape
    buf = util.randn((s, b, hq + 2 * hk, d), dtype, seed=s + d).to(DEV)
    q, k = buf[:, :, :hq], buf[:, :, hq : hq + hk]
    ang = (util.randn((s, 1, 1, d2), torch.float32, seed=d2 + 9) * 5.0).contiguous().to(DEV)
    L = hotpath.lib()
    for backward in (False, True):
        for transpose in (False, True):
            want_q = util.abi_rope_freqs(hotpath, q, ang, backward, transpose)
            want_k = util.abi_rope_freqs(hotpath, k, ang, backward, transpose)
            got_q = util._rope_out(q, transpose)
            got_k = util._rope_out(k, transpose)
            fn = L.nhp_rope_freqs_qk_bwd if backward else L.nhp_rope_freqs_qk_fwd
            rc = fn(got_q.data_ptr(), got_k.data_ptr(), q.data_ptr(), k.data_ptr(), ang.data_ptr(), s, b, hq, hk, d, d2,
                    hotpath.strides4(q), hotpath.strides4(k), hotpath.strides4(got_q), hotpath.strides4(got_k),
                    hotpath.dtype_code(q, "t"), None)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(util.raw_bits(got_q.cpu()), util.raw_bits(want_q.cpu()))
            assert torch.equal(util.raw_bits(got_k.cpu()), util.raw_bits(want_k.cpu()))
    qd, kd = q.detach().clone().requires_grad_(True), k.detach().clone().requires_grad_(True)
    qe, ke = q.detach().clone().requires_grad_(True), k.detach().clone().requires_grad_(True)
    gq, gk = util.randn(q.shape, dtype, seed=1).to(DEV), util.randn(k.shape, dtype, seed=2).to(DEV)
    fq, fk = fused_apply_rotary_pos_emb_qk(qd, kd, ang)
    torch.autograd.backward([fq, fk], [gq, gk])
    oq, ok = fused_apply_rotary_pos_emb(qe, ang), fused_apply_rotary_pos_emb(ke, ang)
    torch.autograd.backward([oq, ok], [gq, gk])
    for a_, b_ in ((fq, oq), (fk, ok), (qd.grad, qe.grad), (kd.grad, ke.grad)):
        assert torch.equal(util.raw_bits(a_.detach().cpu()), util.raw_bits(b_.detach().cpu()))
