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


def near_rounding_boundary(v64, dtype, slack_ulp32=3):
    """Bool tensor: the float64 values v64 lie within `slack_ulp32` fp32 spacings of a point where
    rounding to `dtype` (fp16 / bf16) switches from one representable value to the next. Two fp32
    evaluations of such a value that differ in the last places (device sincosf against libm) may
    round to different `dtype` values; everywhere else they round to the same one."""
    r = v64.to(torch.float32).to(dtype)                       # nearest representable value
    bits = ordered_bits(r)
    def from_ordered(o):
        mag = o.abs().to(torch.int16)
        raw = torch.where(o < 0, mag | torch.tensor(-32768, dtype=torch.int16), mag)
        return raw.view(dtype).double()
    up, down = from_ordered(bits + 1), from_ordered(bits - 1)
    rd = r.double()
    dist = torch.minimum((v64 - (rd + up) / 2).abs(), (v64 - (rd + down) / 2).abs())
    ulp32 = torch.pow(2.0, torch.floor(torch.log2(v64.abs().clamp(min=2.0**-126))) - 23)
    return dist <= slack_ulp32 * ulp32


def rope_freqs_marked(freqs, dtype, backward):
    """[s, 1, 1, d2] bool: elements of a rotary result computed from angles whose cos or sin table
    entry (cos[i], sin[i] in the forward; cos[i], sin[partner(i)] in the backward) sits on a rounding
    boundary of `dtype` in the sense of near_rounding_boundary. fp32 data: nothing is marked (the
    table entries are not narrowed; the comparison is made in fp32 spacings)."""
    f64 = freqs.double()
    if dtype == torch.float32:
        return torch.zeros_like(f64, dtype=torch.bool)
    mc = near_rounding_boundary(torch.cos(f64), dtype)
    ms = near_rounding_boundary(torch.sin(f64), dtype)
    if backward:
        d2 = freqs.size(-1)
        h2 = d2 // 2
        i = torch.arange(d2)
        partner = torch.where(i + h2 < d2, i + h2, i + h2 - d2)   # the reference kernel's index, also for odd d2
        ms = ms[..., partner]
    return mc | ms


def assert_rope_freqs_close(got, want, t, freqs, backward, what="", max_marked_share=0.02):
    """Rotary from angles against the oracle. The only arithmetic that may differ between the two is
    sincosf (device library against libm, both accurate to a few fp32 spacings); the three roundings
    after it are the same. So wherever both table entries of an element are clear of a rounding
    boundary of the data dtype the results must be bit-identical; on the marked elements (a fraction
    of a per cent) one table entry may have rounded the other way, which moves the result by at most
    one spacing of the data dtype at the magnitude of the inputs per entry: 2 spacings at max |t| of
    the head vector. fp32 data: 2 fp32 spacings at that magnitude everywhere."""
    got, want = got.cpu(), want.cpu()
    d2 = freqs.size(-1)
    marked = rope_freqs_marked(freqs.cpu(), got.dtype, backward).expand(got.shape[:-1] + (d2,))
    g, w = got[..., :d2], want[..., :d2]
    scale_ref = t.cpu().float().abs().amax(dim=-1, keepdim=True).expand_as(g.float())
    wide_ok = (g.float() - w.float()).abs() <= 2 * ulp_size(scale_ref.to(got.dtype))
    if got.dtype == torch.float32:
        assert wide_ok.all(), f"{what}: {int((~wide_ok).sum())} fp32 elements out of tolerance"
        return 0.0
    same = raw_bits(g.contiguous()) == raw_bits(w.contiguous())
    bad_clear = ~same & ~marked
    assert not bad_clear.any(), (f"{what}: {int(bad_clear.sum())} elements differ from the oracle although their "
                                 "table entries are clear of a rounding boundary")
    assert (wide_ok | ~marked).all(), f"{what}: a marked element is off by more than two spacings at input magnitude"
    share = float(marked.float().mean())
    assert share <= max_marked_share, f"{what}: {share:.4f} of the elements rest on the wide tolerance"
    return share


BWD_NOISE_SHARES = []  # (what, share of elements beyond 2 ulp, worst ulp distance) of every backward comparison


def assert_softmax_bwd_close(got, want, dy, y, scale, what="", max_noise_share=0.05):
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
    # how much of the result rests on the noise clause rather than on the 2-ulp bound: recorded so that a
    # regression (a kernel that drifts away from the oracle) shows up as a growing share, and bounded
    share = float((~ok_ulp).float().mean()) if got.numel() else 0.0
    BWD_NOISE_SHARES.append((what, share, int(ulp_distance(got, want).max()) if got.numel() else 0))
    assert share <= max_noise_share, f"{what}: {share:.4f} of the elements are beyond 2 ulp (noise clause)"
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
