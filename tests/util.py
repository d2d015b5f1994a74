"""Helpers shared by the tests: bit-level comparisons, tolerances, C-ABI call shims."""
import ctypes
import math

import torch

EPS32 = 2.0**-24


def ordered_bits(t):
    """Map fp16/bf16/fp32 bit patterns to integers that are monotonic in the
    value, so that |a - b| counts representable numbers between a and b
    (+0 and -0 coincide)."""
    if t.dtype == torch.float32:
        raw = t.contiguous().view(torch.int32).to(torch.int64)
        mag = raw & 0x7FFFFFFF
        neg = raw < 0
    else:
        raw = t.contiguous().view(torch.int16).to(torch.int64)
        mag = raw & 0x7FFF
        neg = raw < 0
    return torch.where(neg, -mag, mag)


def ulp_distance(a, b):
    assert a.dtype == b.dtype and a.shape == b.shape
    return (ordered_bits(a) - ordered_bits(b)).abs()


def raw_bits(t):
    if t.dtype == torch.float32:
        return t.contiguous().view(torch.int32)
    return t.contiguous().view(torch.int16)


def assert_ulp_close(got, want, max_ulp, what=""):
    """Every element within max_ulp representable values; NaNs must coincide."""
    got = got.cpu()
    want = want.cpu()
    nan_g, nan_w = torch.isnan(got.float()), torch.isnan(want.float())
    assert torch.equal(nan_g, nan_w), f"{what}: NaN pattern differs"
    d = ulp_distance(got, want)
    d = torch.where(nan_w, torch.zeros_like(d), d)
    worst = int(d.max()) if d.numel() else 0
    if worst > max_ulp:
        idx = int(d.argmax())
        g = got.flatten()[idx].item()
        w = want.flatten()[idx].item()
        raise AssertionError(f"{what}: {worst} ulp apart at flat index {idx}: got {g!r}, want {w!r}")
    return worst


def ulp_size(t):
    """Spacing of the storage dtype at the magnitude of each element (fp32 tensor)."""
    f = t.float().abs()
    if t.dtype == torch.bfloat16:
        mant, emin = 7, -126
    elif t.dtype == torch.float16:
        mant, emin = 10, -14
    else:
        mant, emin = 23, -126
    e = torch.floor(torch.log2(torch.clamp(f, min=2.0**emin)))
    return torch.pow(2.0, e - mant)


def assert_softmax_bwd_close(got, want, dy, y, scale, what=""):
    """Backward tolerance: 2 ulp of the output dtype, plus the rounding noise of
    an fp32 row sum. dx = scale*(g - y*S) cancels, so an S that differs by a few
    fp32 ulp of sum|g| (a different summation order) moves dx by
    scale*|y|*sum|g|*eps32*c, which can exceed 2 ulp of a tiny dx. c = 16
    covers sequential-vs-tree orders for rows of up to 64K elements."""
    got, want = got.cpu(), want.cpu()
    dy, y = dy.cpu().float(), y.cpu().float()
    absg = (dy * y).abs().sum(dim=-1, keepdim=True)
    noise = abs(scale) * (y.abs() * absg + (dy * y).abs()) * 16 * EPS32
    diff = (got.float() - want.float()).abs()
    ok_ulp = ulp_distance(got, want) <= 2
    ok_abs = diff <= noise + 2 * ulp_size(want)
    bad = ~(ok_ulp | ok_abs)
    if bad.any():
        idx = int(bad.flatten().nonzero()[0])
        raise AssertionError(
            f"{what}: element {idx}: got {got.flatten()[idx].item()!r} want {want.flatten()[idx].item()!r} "
            f"noise {noise.flatten()[idx].item():.3e}")
    return int(ulp_distance(got, want).max())


def assert_close_ulp_or_noise(got, want, max_ulp, noise, what=""):
    """Every element within max_ulp representable values of `want`, or within the
    absolute bound `noise` (a tensor: the fp32 rounding noise that the expression
    being tested carries by construction) plus max_ulp spacings."""
    got, want = got.cpu(), want.cpu()
    nan_g, nan_w = torch.isnan(got.float()), torch.isnan(want.float())
    assert torch.equal(nan_g, nan_w), f"{what}: NaN pattern differs"
    d = ulp_distance(got, want)
    diff = (got.float() - want.float()).abs()
    ok = (d <= max_ulp) | (diff <= noise.float() + max_ulp * ulp_size(want)) | nan_w
    if not ok.all():
        idx = int((~ok).flatten().nonzero()[0])
        raise AssertionError(
            f"{what}: element {idx}: got {got.flatten()[idx].item()!r} want {want.flatten()[idx].item()!r} "
            f"({int(d.flatten()[idx])} ulp, allowed noise {noise.float().expand_as(diff).flatten()[idx].item():.3e})")
    return int(torch.where(nan_w, torch.zeros_like(d), d).max()) if d.numel() else 0


def gelu_noise(x, g=None):
    """fp32 rounding noise of the reference's tanh-GeLU expressions at input x (fp32
    tensor): `1 + tanh(u)` and `1 - tanh(u)^2` are formed from a tanh that is only
    known to about 2^-23 absolute, so the forward result carries |x| * 2^-23 of
    noise and the derivative (1 + |x|^3) * 2^-22, whatever their own size."""
    x = x.float().abs()
    if g is None:
        return x * 2.0**-22
    return (1 + x**3) * g.float().abs() * 2.0**-21


def gated_noise(inp, bias, act, want, dy=None):
    """fp32 rounding noise of the expression: a few roundings of the result and, for the erf GeLU,
    the cancellation in 1 + erf(g / sqrt 2) for negative gates (absolute 2^-24 on a factor that
    multiplies g * x), as for the tanh form."""
    x, g = inp.float().chunk(2, -1)
    if bias is not None:
        b1, b2 = bias.float().chunk(2, -1)
        x, g = x + b1, g + b2
    noise = want.abs().float() * 16 * EPS32 + 1e-30
    if dy is not None:
        # 1 - sigmoid(g) in the derivatives cancels for large g: absolute 2^-24 on a factor of dy * x * (1 + |g|)
        d = dy.float().abs()
        noise = noise + torch.cat([torch.zeros_like(d), d * x.abs() * (1 + g.abs())], -1) * 4 * EPS32
    if act == "geglu":
        tail = (x * g).abs() * 4 * EPS32
        if dy is None:
            noise = noise + tail
        else:
            d = dy.float().abs()
            noise = noise + torch.cat([d * g.abs(), d * x.abs() * (1 + g * g)], -1) * 4 * EPS32
    return noise



# ---------------------------------------------------------------------------
# direct C-ABI calls on torch GPU tensors
# ---------------------------------------------------------------------------
def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def abi_causal_fwd(hp, x, scale):
    y = torch.empty_like(x)
    rc = hp.lib().nhp_causal_softmax_fwd(y.data_ptr(), x.data_ptr(), scale, x.size(0), x.size(1),
                                         hp.dtype_code(x, "t"), _stream())
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return y


def abi_causal_bwd(hp, dy, y, scale, inplace=False):
    dx = dy if inplace else torch.empty_like(dy)
    rc = hp.lib().nhp_causal_softmax_bwd(dx.data_ptr(), dy.data_ptr(), y.data_ptr(), scale, dy.size(0),
                                         dy.size(1), hp.dtype_code(dy, "t"), _stream())
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return dx


def abi_masked_fwd(hp, x, mask, scale):
    y = torch.empty_like(x)
    b, np_, sq, sk = x.shape
    rc = hp.lib().nhp_masked_softmax_fwd(y.data_ptr(), x.data_ptr(), mask.data_ptr(), scale, b, np_, sq, sk,
                                         mask.size(0), hp.dtype_code(x, "t"), _stream())
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return y


def abi_masked_bwd(hp, dy, y, scale, inplace=False):
    dx = dy if inplace else torch.empty_like(dy)
    sk = dy.size(-1)
    rc = hp.lib().nhp_masked_softmax_bwd(dx.data_ptr(), dy.data_ptr(), y.data_ptr(), scale, dy.numel() // sk,
                                         sk, hp.dtype_code(dy, "t"), _stream())
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return dx


def _rope_out(t, transpose):
    s, b, h, d = t.shape
    if transpose:
        return torch.empty((b, s, h, d), dtype=t.dtype, device=t.device).transpose(0, 1)
    return torch.empty((s, b, h, d), dtype=t.dtype, device=t.device)


def abi_rope_cached(hp, t, cos, sin, backward=False, transpose=False):
    out = _rope_out(t, transpose)
    s, b, h, d = t.shape
    fn = hp.lib().nhp_rope_cached_bwd if backward else hp.lib().nhp_rope_cached_fwd
    rc = fn(out.data_ptr(), t.data_ptr(), cos.data_ptr(), sin.data_ptr(), s, b, h, d, cos.size(-1),
            hp.strides4(t), hp.strides4(out), hp.dtype_code(t, "t"), hp.dtype_code(cos, "c"), _stream())
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return out


def abi_rope_freqs(hp, t, freqs, backward=False, transpose=False):
    out = _rope_out(t, transpose)
    s, b, h, d = t.shape
    fn = hp.lib().nhp_rope_freqs_bwd if backward else hp.lib().nhp_rope_freqs_fwd
    rc = fn(out.data_ptr(), t.data_ptr(), freqs.data_ptr(), s, b, h, d, freqs.size(-1), hp.strides4(t),
            hp.strides4(out), hp.dtype_code(t, "t"), _stream())
    assert rc == 0, hp.lib().nhp_status_string(rc)
    return out


def randn(shape, dtype, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def padding_mask(b, sq, sk, seed, full_batch=None, lo=None):
    """[b,1,sq,sk] bool: keys at or beyond a per-sequence valid length are
    masked; sequence `full_batch` is masked entirely."""
    g = torch.Generator().manual_seed(seed)
    lo = max(1, sk // 4) if lo is None else lo
    valid = torch.randint(lo, sk + 1, (b,), generator=g)
    k = torch.arange(sk)
    m = (k[None, :] >= valid[:, None])[:, None, None, :].expand(b, 1, sq, sk).contiguous()
    if full_batch is not None:
        m[full_batch] = True
    return m
