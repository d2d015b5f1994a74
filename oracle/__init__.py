"""TEST INFRASTRUCTURE -- NOT PART OF THE PRODUCT.

CPU oracle for the fused softmax / rotary hot path. Two restatements live here:

* ``kernel_semantics.c`` (this module's ctypes wrappers): what the reference's
  CUDA kernels compute, element by element, in plain C.
* ``fallback_semantics.py``: the reference's own torch fallback
  (``FusedScaleMaskSoftmax.forward_torch_softmax``, the eager rotary functions
  and the ``RotaryEmbedding`` cache recipe).

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg
may import this package, and only as the checker. The product package never
does; it raises when its HIP library is missing.

All wrappers take and return CPU ``torch`` tensors.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

DT_F16, DT_BF16, DT_F32 = 0, 1, 2
_DT = {torch.float16: DT_F16, torch.bfloat16: DT_BF16, torch.float32: DT_F32}


def build(force=False):
    """Compile liboracle.so with gcc (a few hundred milliseconds)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, f32, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_int
        L.oracle_causal_softmax_fwd.argtypes = [vp, vp, f32, i64, i64, ci]
        L.oracle_causal_softmax_ex_fwd.argtypes = [vp, vp, f32, i64, i64, i64, vp, vp, vp, i64, ci]
        L.oracle_softmax_ex_bwd.argtypes = [vp, vp, vp, f32, i64, i64, i64, ci, i64, vp, i64, ci]
        L.oracle_masked_softmax_fwd.argtypes = [vp, vp, vp, f32, i64, i64, i64, i64, i64, ci]
        L.oracle_softmax_bwd.argtypes = [vp, vp, vp, f32, i64, i64, i64, ci, ci]
        L.oracle_batch_per_block.argtypes = [i64, ci]
        L.oracle_bias_gelu_fwd.argtypes = [vp, vp, vp, i64, i64, ci]
        L.oracle_bias_gelu_bwd.argtypes = [vp, vp, vp, vp, i64, i64, ci]
        L.oracle_column_sum.argtypes = [vp, vp, i64, i64, ci]
        L.oracle_bias_add_residual.argtypes = [vp, vp, vp, vp, i64, i64, ci]
        u64 = ctypes.c_uint64
        pu32 = ctypes.POINTER(ctypes.c_uint32)
        L.oracle_philox4x32_10.argtypes = [pu32, pu32, pu32]
        L.oracle_philox4x32_10.restype = None
        L.oracle_dropout_mask.argtypes = [vp, i64, f32, u64, u64]
        L.oracle_bias_dropout_add.argtypes = [vp, vp, vp, vp, i64, i64, f32, u64, u64, ci]
        L.oracle_causal_softmax_dropout_fwd.argtypes = [vp, vp, vp, f32, i64, i64, i64, f32, u64, u64, ci]
        L.oracle_causal_softmax_dropout_bwd.argtypes = [vp, vp, vp, f32, i64, i64, i64, f32, u64, u64, ci]
        L.oracle_gated_act_fwd.argtypes = [vp, vp, vp, i64, i64, ci, ci]
        L.oracle_gated_act_bwd.argtypes = [vp, vp, vp, vp, i64, i64, ci, ci]
        L.oracle_layernorm_fwd.argtypes = [vp, vp, vp, vp, vp, vp, f32, i64, i64, ci, ci]
        L.oracle_layernorm_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, ci, ci]
        L.oracle_layernorm_pair_dx.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, ci, ci]
        L.oracle_rmsnorm_fwd.argtypes = [vp, vp, vp, vp, vp, f32, ci, i64, i64, i64, ci, ci]
        L.oracle_rmsnorm_bwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, f32, ci, i64, i64, i64, ci, ci]
        p64 = ctypes.POINTER(i64)
        L.oracle_rope_cached.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, p64, p64, ci, ci, ci]
        L.oracle_rope_freqs.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, p64, p64, ci, ci]
        L.oracle_float_to_bf16.argtypes = [f32]
        L.oracle_float_to_bf16.restype = ctypes.c_uint16
        L.oracle_float_to_f16.argtypes = [f32]
        L.oracle_float_to_f16.restype = ctypes.c_uint16
        L.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_float.restype = f32
        L.oracle_f16_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_float.restype = f32
        _lib = L
    return _lib


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with code {rc}")


def _cpu_contig(t):
    assert t.device.type == "cpu", "the oracle works on CPU tensors"
    return t.contiguous()


def _key_lengths(key_lengths, attn_batches, heads):
    """int32 [batch] tensor and the heads-per-batch-entry divisor for the C side."""
    if key_lengths is None:
        return None, None, heads
    kl = _cpu_contig(key_lengths.to(torch.int32))
    if heads is None:
        heads = attn_batches // kl.numel()
    assert kl.numel() * heads == attn_batches, "key_lengths needs attn_batches == batch * heads"
    return kl, kl.data_ptr(), heads


def causal_softmax_fwd(x, scale, window=None, alibi_slopes=None, bias=None, key_lengths=None):
    """x: [attn_batches, s, s] fp16/bf16 -> probabilities, same shape and dtype.
    window: sliding-window width or None; alibi_slopes: fp32 [heads] or None;
    bias: [heads, s, s] in x.dtype or None; key_lengths: integer [batch] or None
    (attn_batches = batch * heads, keys >= the length are padding)."""
    assert x.dim() == 3 and x.size(1) == x.size(2)
    x = _cpu_contig(x)
    y = torch.empty_like(x)
    sl_ptr, heads = None, None
    if alibi_slopes is not None:
        alibi_slopes = _cpu_contig(alibi_slopes.float())
        sl_ptr, heads = alibi_slopes.data_ptr(), alibi_slopes.numel()
        assert x.size(0) % heads == 0
    b_ptr = None
    if bias is not None:
        bias = _cpu_contig(bias)
        assert bias.dtype == x.dtype and bias.shape[1:] == x.shape[1:]
        assert alibi_slopes is None or bias.size(0) == heads
        b_ptr, heads = bias.data_ptr(), bias.size(0)
        assert x.size(0) % heads == 0
    kl, kl_ptr, heads = _key_lengths(key_lengths, x.size(0), heads)
    _check(lib().oracle_causal_softmax_ex_fwd(y.data_ptr(), x.data_ptr(), float(scale), x.size(0), x.size(1),
                                              -1 if window is None else int(window), sl_ptr, b_ptr, kl_ptr,
                                              heads or 1, _DT[x.dtype]), "causal_softmax_fwd")
    return y


def prepared_masked_inputs(x, mask, alibi_slopes=None, bias=None, key_lengths=None):
    """What the caller of the padding-mask softmax does to its operands beforehand
    (megatron/model/transformer.py:580-588), as eager torch statements in the scores' dtype:
    `attention_scores += rpe` (bias [np, sq, sk] or [1, np, sq, sk]), then AliBi.forward
    (megatron/model/positional_embeddings.py:219-257, sq == sk), and the padding keys
    k >= key_lengths[b] merged into the mask. Returns (scores, mask [b or 1, 1, sq, sk] bool)."""
    from . import fallback_semantics as fb

    b, np_, sq, sk = x.shape
    if bias is not None:
        x = x + bias.view(1, np_, sq, sk)
    if alibi_slopes is not None:
        assert sq == sk
        x = fb.alibi_add(x, alibi_slopes)
    m = mask.bool() if mask.dtype != torch.bool else mask
    if key_lengths is not None:
        assert key_lengths.numel() == b
        keys = torch.arange(sk)
        m = m | (keys.view(1, 1, 1, sk) >= key_lengths.clamp(min=0).view(b, 1, 1, 1))
    return x, m


def masked_softmax_fwd(x, mask, scale, alibi_slopes=None, bias=None, key_lengths=None):
    """x: [b, np, sq, sk]; mask: [1 or b, 1, sq, sk] bool/uint8 (value 1 masks).
    alibi_slopes (fp32 [np]), bias ([np, sq, sk] in x.dtype) and key_lengths (integer [b]) are applied
    as prepared_masked_inputs does, i.e. the result is the plain softmax of the prepared operands."""
    assert x.dim() == 4 and mask.dim() == 4
    if alibi_slopes is not None or bias is not None or key_lengths is not None:
        x, mask = prepared_masked_inputs(x, mask, alibi_slopes, bias, key_lengths)
    x = _cpu_contig(x)
    m = _cpu_contig(mask).view(torch.uint8) if mask.dtype == torch.bool else _cpu_contig(mask)
    assert m.dtype == torch.uint8
    b, np_, sq, sk = x.shape
    assert m.size(1) == 1 and m.size(2) == sq and m.size(3) == sk
    y = torch.empty_like(x)
    _check(lib().oracle_masked_softmax_fwd(y.data_ptr(), x.data_ptr(), m.data_ptr(), float(scale), b, np_, sq,
                                           sk, m.size(0), _DT[x.dtype]), "masked_softmax_fwd")
    return y


def softmax_bwd(dy, y, scale, causal, window=None, key_lengths=None):
    """Returns dx (a new tensor). dy, y: [..., rows_per_matrix, n]; key_lengths
    (causal only): integer [batch] with dy [batch * heads, s, s]."""
    dy = _cpu_contig(dy)
    y = _cpu_contig(y)
    assert dy.shape == y.shape and dy.dtype == y.dtype
    n = dy.size(-1)
    rows = dy.numel() // max(n, 1)
    dx = torch.empty_like(dy)
    kl, kl_ptr, heads = _key_lengths(key_lengths, rows // max(dy.size(-2), 1), None)
    _check(lib().oracle_softmax_ex_bwd(dx.data_ptr(), dy.data_ptr(), y.data_ptr(), float(scale), rows, n,
                                       dy.size(-2), 1 if causal else 0, -1 if window is None else int(window),
                                       kl_ptr, heads or 1, _DT[dy.dtype]), "softmax_bwd")
    return dx


def batch_per_block(sk, warp=64):
    return lib().oracle_batch_per_block(int(sk), int(warp))


def _strides4(t):
    return (ctypes.c_int64 * 4)(*t.stride())


def _rope_out(t, transpose_output):
    s, b, h, d = t.shape
    if transpose_output:
        return torch.empty((b, s, h, d), dtype=t.dtype).transpose(0, 1)
    return torch.empty((s, b, h, d), dtype=t.dtype)


def rope_cached(t, cos, sin, backward=False, transpose_output=False):
    """t: [s,b,h,d] (any strides); cos, sin: [s,1,1,d2] fp32 or t.dtype."""
    assert t.device.type == "cpu" and t.dim() == 4
    cos = _cpu_contig(cos)
    sin = _cpu_contig(sin)
    s, b, h, d = t.shape
    d2 = cos.size(3)
    out = _rope_out(t, transpose_output)
    _check(lib().oracle_rope_cached(out.data_ptr(), t.data_ptr(), cos.data_ptr(), sin.data_ptr(), s, b, h, d,
                                    d2, _strides4(t), _strides4(out), _DT[t.dtype], _DT[cos.dtype],
                                    1 if backward else 0), "rope_cached")
    return out


def rope_freqs(t, freqs, backward=False, transpose_output=False):
    """t: [s,b,h,d]; freqs: [s,1,1,d2] fp32 angles."""
    assert t.device.type == "cpu" and t.dim() == 4 and freqs.dtype == torch.float32
    freqs = _cpu_contig(freqs)
    s, b, h, d = t.shape
    d2 = freqs.size(3)
    out = _rope_out(t, transpose_output)
    _check(lib().oracle_rope_freqs(out.data_ptr(), t.data_ptr(), freqs.data_ptr(), s, b, h, d, d2,
                                   _strides4(t), _strides4(out), _DT[t.dtype], 1 if backward else 0),
           "rope_freqs")
    return out


# ---------------------------------------------------------------------------
# element-wise layer functions (layer_semantics.c)
# ---------------------------------------------------------------------------
def _rows_cols(t):
    cols = t.size(-1)
    return t.numel() // max(cols, 1), cols


def _opt_ptr(t, like, what):
    if t is None:
        return None, None
    t = _cpu_contig(t)
    assert t.dtype == like.dtype, what
    return t, t.data_ptr()


def bias_gelu_fwd(y, bias=None):
    """gelu_tanh(bias + y); y: [..., cols], bias: [cols] or None."""
    y = _cpu_contig(y)
    out = torch.empty_like(y)
    rows, cols = _rows_cols(y)
    bias, bp = _opt_ptr(bias, y, "bias dtype")
    _check(lib().oracle_bias_gelu_fwd(out.data_ptr(), y.data_ptr(), bp, rows, cols, _DT[y.dtype]), "bias_gelu_fwd")
    return out


def bias_gelu_bwd(g, y, bias=None):
    """gelu_tanh'(bias + y) * g."""
    y = _cpu_contig(y)
    g = _cpu_contig(g)
    assert g.shape == y.shape and g.dtype == y.dtype
    dx = torch.empty_like(y)
    rows, cols = _rows_cols(y)
    bias, bp = _opt_ptr(bias, y, "bias dtype")
    _check(lib().oracle_bias_gelu_bwd(dx.data_ptr(), g.data_ptr(), y.data_ptr(), bp, rows, cols, _DT[y.dtype]),
           "bias_gelu_bwd")
    return dx


def column_sum(t):
    """Sum over all leading dimensions, fp32 accumulation, result [cols] in t.dtype."""
    t = _cpu_contig(t)
    rows, cols = _rows_cols(t)
    out = torch.empty(cols, dtype=t.dtype)
    _check(lib().oracle_column_sum(out.data_ptr(), t.data_ptr(), rows, cols, _DT[t.dtype]), "column_sum")
    return out


def bias_add_residual(x, bias=None, residual=None):
    """residual + (x + bias), one rounding."""
    x = _cpu_contig(x)
    out = torch.empty_like(x)
    rows, cols = _rows_cols(x)
    bias, bp = _opt_ptr(bias, x, "bias dtype")
    residual, rp = _opt_ptr(residual, x, "residual dtype")
    _check(lib().oracle_bias_add_residual(out.data_ptr(), x.data_ptr(), bp, rp, rows, cols, _DT[x.dtype]),
           "bias_add_residual")
    return out


# ---------------------------------------------------------------------------
# LayerNorm / RMSNorm (layer_semantics.c)
# ---------------------------------------------------------------------------
def _param(t, x):
    """(tensor kept alive, pointer, dtype code) of an optional [cols] parameter: fp32 or x.dtype."""
    if t is None:
        return None, None, None
    t = _cpu_contig(t)
    assert t.dtype in (x.dtype, torch.float32) and t.numel() == x.size(-1)
    return t, t.data_ptr(), _DT[t.dtype]


def _param_code(x, *codes):
    codes = {c for c in codes if c is not None}
    assert len(codes) <= 1, "all parameters must share one dtype"
    return codes.pop() if codes else _DT[x.dtype]


def layernorm_fwd(x, gamma=None, beta=None, eps=1e-5):
    """Returns (y, mean, rstd); x: [..., cols]."""
    x = _cpu_contig(x)
    rows, cols = _rows_cols(x)
    y = torch.empty_like(x)
    mean = torch.empty(rows, dtype=torch.float32)
    rstd = torch.empty(rows, dtype=torch.float32)
    gamma, gp, gc = _param(gamma, x)
    beta, bp, bc = _param(beta, x)
    _check(lib().oracle_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), gp, bp,
                                      float(eps), rows, cols, _DT[x.dtype], _param_code(x, gc, bc)), "layernorm_fwd")
    return y, mean, rstd


def layernorm_bwd(dy, x, mean, rstd, gamma=None, param_dtype=None):
    """Returns (dx, dgamma, dbeta); the parameter gradients come in param_dtype (default: gamma's, else x's)."""
    x = _cpu_contig(x)
    dy = _cpu_contig(dy)
    rows, cols = _rows_cols(x)
    gamma, gp, gc = _param(gamma, x)
    pdt = param_dtype or (gamma.dtype if gamma is not None else x.dtype)
    dx = torch.empty_like(x)
    dg = torch.empty(cols, dtype=pdt)
    db = torch.empty(cols, dtype=pdt)
    mean, rstd = _cpu_contig(mean.float()), _cpu_contig(rstd.float())
    _check(lib().oracle_layernorm_bwd(dx.data_ptr(), dg.data_ptr(), db.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                      mean.data_ptr(), rstd.data_ptr(), gp, rows, cols, _DT[x.dtype], _DT[pdt]),
           "layernorm_bwd")
    return dx, dg, db


def rmsnorm_fwd(x, scale=None, offset=None, eps=1e-8, eps_mode=1, stat_cols=None):
    """Returns (y, inv). eps_mode 1: x / (rms + eps) (the Python RMSNorm class); 0: x * rsqrt(mean(x^2) + eps);
    2: x / max(||x||, eps) (ScaleNorm). stat_cols: leading columns the statistic is taken over (default: all)."""
    x = _cpu_contig(x)
    rows, cols = _rows_cols(x)
    y = torch.empty_like(x)
    inv = torch.empty(rows, dtype=torch.float32)
    scale, sp, sc = _param(scale, x)
    offset, op, oc = _param(offset, x)
    _check(lib().oracle_rmsnorm_fwd(y.data_ptr(), inv.data_ptr(), x.data_ptr(), sp, op, float(eps), int(eps_mode),
                                    rows, cols, cols if stat_cols is None else int(stat_cols), _DT[x.dtype],
                                    _param_code(x, sc, oc)), "rmsnorm_fwd")
    return y, inv


def rmsnorm_bwd(dy, x, inv, scale=None, eps=1e-8, eps_mode=1, param_dtype=None, stat_cols=None):
    """Returns (dx, dscale, doffset)."""
    x = _cpu_contig(x)
    dy = _cpu_contig(dy)
    rows, cols = _rows_cols(x)
    scale, sp, sc = _param(scale, x)
    pdt = param_dtype or (scale.dtype if scale is not None else x.dtype)
    dx = torch.empty_like(x)
    ds = torch.empty(cols, dtype=pdt)
    do = torch.empty(cols, dtype=pdt)
    inv = _cpu_contig(inv.float())
    _check(lib().oracle_rmsnorm_bwd(dx.data_ptr(), ds.data_ptr(), do.data_ptr(), dy.data_ptr(), x.data_ptr(),
                                    inv.data_ptr(), sp, float(eps), int(eps_mode), rows, cols,
                                    cols if stat_cols is None else int(stat_cols), _DT[x.dtype], _DT[pdt]),
           "rmsnorm_bwd")
    return dx, ds, do


# ---------------------------------------------------------------------------
# gated activations (layer_semantics.c)
# ---------------------------------------------------------------------------
GATE_ACTS = {"swiglu": 0, "geglu": 1, "reglu": 2, "glu": 3, "bilinear": 4}


def gated_act_fwd(inp, act, bias=None):
    """act(gate) * x with x, gate = inp.chunk(2, -1) (+ the halves of bias); act: a key of GATE_ACTS."""
    inp = _cpu_contig(inp)
    assert inp.size(-1) % 2 == 0
    f = inp.size(-1) // 2
    rows = inp.numel() // max(2 * f, 1)
    out = torch.empty(inp.shape[:-1] + (f,), dtype=inp.dtype)
    bias, bp = _opt_ptr(bias, inp, "bias dtype")
    _check(lib().oracle_gated_act_fwd(out.data_ptr(), inp.data_ptr(), bp, rows, f, GATE_ACTS[act], _DT[inp.dtype]),
           "gated_act_fwd")
    return out


def gated_act_bwd(dy, inp, act, bias=None):
    """Gradient with respect to inp (the bias gradient is its column sum)."""
    inp = _cpu_contig(inp)
    dy = _cpu_contig(dy)
    f = inp.size(-1) // 2
    rows = inp.numel() // max(2 * f, 1)
    assert dy.shape == inp.shape[:-1] + (f,) and dy.dtype == inp.dtype
    din = torch.empty_like(inp)
    bias, bp = _opt_ptr(bias, inp, "bias dtype")
    _check(lib().oracle_gated_act_bwd(din.data_ptr(), dy.data_ptr(), inp.data_ptr(), bp, rows, f, GATE_ACTS[act],
                                      _DT[inp.dtype]), "gated_act_bwd")
    return din


# ---------------------------------------------------------------------------
# dropout (layer_semantics.c)
# ---------------------------------------------------------------------------
def philox4x32_10(counter, key):
    """The four 32-bit output words for a 4-word counter and a 2-word key."""
    c = (ctypes.c_uint32 * 4)(*counter)
    k = (ctypes.c_uint32 * 2)(*key)
    out = (ctypes.c_uint32 * 4)()
    lib().oracle_philox4x32_10(c, k, out)
    return list(out)


def dropout_mask(n, p, seed, offset=0):
    """bool [n]: which elements (by flat index) are kept."""
    keep = torch.empty(max(n, 1), dtype=torch.uint8)
    _check(lib().oracle_dropout_mask(keep.data_ptr(), n, float(p), int(seed), int(offset)), "dropout_mask")
    return keep[:n].bool()


def bias_dropout_add(x, bias, residual, p, seed, offset=0):
    """residual + keep * (x + bias) / (1 - p) with the mask of dropout_mask."""
    x = _cpu_contig(x)
    out = torch.empty_like(x)
    rows, cols = _rows_cols(x)
    bias, bp = _opt_ptr(bias, x, "bias dtype")
    residual, rp = _opt_ptr(residual, x, "residual dtype")
    _check(lib().oracle_bias_dropout_add(out.data_ptr(), x.data_ptr(), bp, rp, rows, cols, float(p), int(seed),
                                         int(offset), _DT[x.dtype]), "bias_dropout_add")
    return out


def causal_softmax_dropout_fwd(x, scale, p, seed, offset=0, window=None, alibi_slopes=None, bias=None, key_lengths=None):
    """Returns (dropped, y): the probabilities y and dropout(y) with the mask of dropout_mask over x's flat index.
    With AliBi slopes, a bias or key lengths: causal_softmax_fwd with them, then the dropout of its stored result."""
    assert x.dim() == 3 and x.size(1) == x.size(2)
    x = _cpu_contig(x)
    if alibi_slopes is not None or bias is not None or key_lengths is not None:
        y = causal_softmax_fwd(x, scale, window, alibi_slopes, bias, key_lengths)
        return _dropout_of_stored(y, p, seed, offset), y
    y, dropped = torch.empty_like(x), torch.empty_like(x)
    _check(lib().oracle_causal_softmax_dropout_fwd(dropped.data_ptr(), y.data_ptr(), x.data_ptr(), float(scale), x.size(0),
                                                   x.size(1), -1 if window is None else int(window), float(p), int(seed),
                                                   int(offset), _DT[x.dtype]), "causal_softmax_dropout_fwd")
    return dropped, y


def causal_softmax_dropout_bwd(dy, y, scale, p, seed, offset=0, window=None, key_lengths=None):
    """Gradient with respect to the scores, given the gradient of dropout(y)."""
    dy, y = _cpu_contig(dy), _cpu_contig(y)
    if key_lengths is not None:
        return softmax_bwd(_dropout_of_stored(dy, p, seed, offset), y, scale, True, window, key_lengths)
    dx = torch.empty_like(dy)
    _check(lib().oracle_causal_softmax_dropout_bwd(dx.data_ptr(), dy.data_ptr(), y.data_ptr(), float(scale), dy.size(0),
                                                   dy.size(1), -1 if window is None else int(window), float(p), int(seed),
                                                   int(offset), _DT[dy.dtype]), "causal_softmax_dropout_bwd")
    return dx


def _dropout_of_stored(t, p, seed, offset):
    """keep ? t / (1 - p) : 0 on the stored values of t, rounded to t's dtype (fp32 product, as in
    oracle_causal_softmax_dropout_fwd), with the mask of dropout_mask over t's flat index."""
    import numpy as np

    keep = dropout_mask(t.numel(), p, seed, offset).view(t.shape)
    ds = torch.tensor(np.float32(1.0 / (1.0 - float(np.float32(p)))))
    scaled = (t.float() * ds).to(t.dtype)
    return torch.where(keep, scaled, torch.zeros_like(scaled))


def masked_softmax_dropout_fwd(x, mask, scale, p, seed, offset=0, alibi_slopes=None, bias=None, key_lengths=None):
    """Returns (dropped, y) for the padding-mask softmax followed by attention dropout
    (megatron/model/transformer.py:588-593): the composition of masked_softmax_fwd and the dropout of its
    stored result, the mask taken over the flat index of the [b, np, sq, sk] tensor."""
    y = masked_softmax_fwd(x, mask, scale, alibi_slopes, bias, key_lengths)
    return _dropout_of_stored(y, p, seed, offset), y


def masked_softmax_dropout_bwd(dy, y, scale, p, seed, offset=0):
    """Gradient with respect to the scores, given the gradient of dropout(y): the dropout backward stored in
    the storage type, then the (unmasked) softmax backward."""
    dy, y = _cpu_contig(dy), _cpu_contig(y)
    return softmax_bwd(_dropout_of_stored(dy, p, seed, offset), y, scale, False)


def layernorm_pair_fwd(x, gamma1, beta1, gamma2, beta2, eps=1e-5):
    """Two LayerNorms of one input: (y1, y2, mean, rstd), the statistics shared."""
    y1, mean, rstd = layernorm_fwd(x, gamma1, beta1, eps)
    y2, _, _ = layernorm_fwd(x, gamma2, beta2, eps)
    return y1, y2, mean, rstd


def layernorm_pair_bwd(dy1, dy2, x, mean, rstd, gamma1, gamma2):
    """(dx, dgamma1, dbeta1, dgamma2, dbeta2): dx from g = dy1 * gamma1 + dy2 * gamma2 with one rounding, the
    parameter gradients of the two single LayerNorms."""
    x, dy1, dy2 = _cpu_contig(x), _cpu_contig(dy1), _cpu_contig(dy2)
    rows, cols = _rows_cols(x)
    gamma1, g1p, _ = _param(gamma1, x)
    gamma2, g2p, _ = _param(gamma2, x)
    pdt = gamma1.dtype if gamma1 is not None else (gamma2.dtype if gamma2 is not None else x.dtype)
    if gamma1 is not None and gamma2 is not None:
        assert gamma1.dtype == gamma2.dtype
    mean, rstd = _cpu_contig(mean.float()), _cpu_contig(rstd.float())
    dx = torch.empty_like(x)
    _check(lib().oracle_layernorm_pair_dx(dx.data_ptr(), dy1.data_ptr(), dy2.data_ptr(), x.data_ptr(), mean.data_ptr(),
                                          rstd.data_ptr(), g1p, g2p, rows, cols, _DT[x.dtype], _DT[pdt]),
           "layernorm_pair_dx")
    _, dg1, db1 = layernorm_bwd(dy1, x, mean, rstd, gamma1, param_dtype=pdt)
    _, dg2, db2 = layernorm_bwd(dy2, x, mean, rstd, gamma2, param_dtype=pdt)
    return dx, dg1, db1, dg2, db2


def bias_add_residual_pair(x1, bias1, x2, bias2, residual):
    """residual + ((x1 + bias1) + (x2 + bias2)) as the parallel-residual layer's three bias_dropout_add calls with
    dropout off, each evaluated in fp32 and rounded once (bias_add_residual): t1 = x1 + bias1 (skipped without
    bias1), t3 = t1 + (x2 + bias2), result = residual + t3."""
    t1 = x1 if bias1 is None else bias_add_residual(x1, bias1, None)
    return bias_add_residual(bias_add_residual(x2, bias2, t1), None, residual)
