"""Extension-module surface of the fused rotary positional embedding.

Same functions as the reference's pybind module
(megatron/fused_kernels/fused_rotary_positional_embedding.cpp:129-139), served
by libneox_hotpath.so. The input may have arbitrary strides; the output is a
new contiguous [s,b,h,d] tensor, or [b,s,h,d] storage viewed as [s,b,h,d] when
``transpose_output`` is set. Launches are asynchronous on the current stream.
"""
import torch

from megatron.fused_kernels import _hotpath as _hp

_FLOATS = (torch.float16, torch.bfloat16, torch.float32)


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _new_output(t, transpose_output):
    s, b, h, d = t.shape
    if transpose_output:
        return torch.empty((b, s, h, d), dtype=t.dtype, device=t.device).transpose(0, 1)
    return torch.empty((s, b, h, d), dtype=t.dtype, device=t.device)


def _run_freqs(name, fn, t, freqs, transpose_output, what):
    # argument checks of fused_rotary_positional_embedding.cpp:39-73
    _check(t.dim() == 4, "expected 4D tensor")
    _check(freqs.dim() == 4, "expected 4D tensor")
    _check(t.size(0) == freqs.size(0), f"expected {what} and freqs tensor have the same sequence length")
    _check(freqs.size(1) == 1 and freqs.size(2) == 1,
           "expected the second and third dims of the freqs tensor equal 1")
    _check(t.size(3) >= freqs.size(3),
           f"expected the last dim of the {what} tensor equals or is greater than the freqs tensor")
    _check(freqs.dtype == torch.float32, "Dtype of the freqs tensor must be float")
    _check(t.dtype in _FLOATS, f"{name}: unsupported dtype {t.dtype}")
    _hp.require_gpu(t, name)
    _hp.require_gpu(freqs, name)
    f = freqs.contiguous()
    out = _new_output(t, transpose_output)
    s, b, h, d = t.shape
    with _hp.device_guard(t):
        rc = fn(out.data_ptr(), t.data_ptr(), f.data_ptr(), s, b, h, d, f.size(3), _hp.strides4(t),
                _hp.strides4(out), _hp.dtype_code(t, name), _hp.stream_of(t))
    _hp.check(rc, name)
    return out


def _run_cached(name, fn, t, cos, sin, transpose_output, what):
    # argument checks of fused_rotary_positional_embedding.cpp:75-125
    _check(t.dim() == 4, "expected 4D tensor")
    _check(cos.dim() == 4, "expected 4D tensor")
    _check(sin.dim() == 4, "expected 4D tensor")
    _check(t.size(0) == cos.size(0), f"expected {what} and cos tensor have the same sequence length")
    _check(t.size(0) == sin.size(0), f"expected {what} and sin tensor have the same sequence length")
    _check(cos.size(1) == 1 and cos.size(2) == 1, "expected the second and third dims of the cos tensor equal 1")
    _check(sin.size(1) == 1 and sin.size(2) == 1, "expected the second and third dims of the sin tensor equal 1")
    _check(cos.size(3) == sin.size(3), "expected cos and sin tensor have the same last dim")
    _check(t.size(3) >= cos.size(3),
           f"expected the last dim of the {what} tensor equals or is greater than the cos tensor")
    _check(cos.dtype == sin.dtype, "expected cos and sin tensor have the same dtype")
    _check(t.dtype in _FLOATS, f"{name}: unsupported dtype {t.dtype}")
    _check(cos.dtype == torch.float32 or cos.dtype == t.dtype,
           f"{name}: cos/sin must be float32 or have the dtype of the input")
    _hp.require_gpu(t, name)
    _hp.require_gpu(cos, name)
    _hp.require_gpu(sin, name)
    c = cos.contiguous()
    sn = sin.contiguous()
    out = _new_output(t, transpose_output)
    s, b, h, d = t.shape
    with _hp.device_guard(t):
        rc = fn(out.data_ptr(), t.data_ptr(), c.data_ptr(), sn.data_ptr(), s, b, h, d, c.size(3),
                _hp.strides4(t), _hp.strides4(out), _hp.dtype_code(t, name), _hp.dtype_code(c, name),
                _hp.stream_of(t))
    _hp.check(rc, name)
    return out


def forward(input, freqs, transpose_output):
    """Rotate ``input`` [s,b,h,d] by the fp32 angles ``freqs`` [s,1,1,d2]."""
    return _run_freqs("fused_rotary_positional_embedding.forward", _hp.lib().nhp_rope_freqs_fwd, input, freqs,
                      transpose_output, "input")


def backward(output_grads, freqs, transpose_output):
    """Gradient of ``forward`` w.r.t. its input."""
    return _run_freqs("fused_rotary_positional_embedding.backward", _hp.lib().nhp_rope_freqs_bwd, output_grads,
                      freqs, transpose_output, "output_grads")


def forward_cached(input, cos, sin, transpose_output):
    """Rotate ``input`` [s,b,h,d] with cached ``cos``/``sin`` [s,1,1,d2]."""
    return _run_cached("fused_rotary_positional_embedding.forward_cached", _hp.lib().nhp_rope_cached_fwd, input,
                       cos, sin, transpose_output, "input")


def backward_cached(output_grads, cos, sin, transpose_output):
    """Gradient of ``forward_cached`` w.r.t. its input."""
    return _run_cached("fused_rotary_positional_embedding.backward_cached", _hp.lib().nhp_rope_cached_bwd,
                       output_grads, cos, sin, transpose_output, "output_grads")


def _run_cached_qk(name, fn, q, k, cos, sin, transpose_output, out=None):
    for t, what in ((q, "q"), (k, "k")):
        _check(t.dim() == 4, "expected 4D tensor")
        _check(t.size(0) == cos.size(0), f"expected {what} and cos tensor have the same sequence length")
        _check(t.size(3) >= cos.size(3),
               f"expected the last dim of the {what} tensor equals or is greater than the cos tensor")
        _check(t.dtype in _FLOATS, f"{name}: unsupported dtype {t.dtype}")
        _hp.require_gpu(t, name)
    _check(cos.dim() == 4 and sin.dim() == 4, "expected 4D tensor")
    _check(cos.shape == sin.shape, "expected cos and sin tensor have the same shape")
    _check(cos.size(1) == 1 and cos.size(2) == 1, "expected the second and third dims of the cos tensor equal 1")
    _check(cos.dtype == sin.dtype, "expected cos and sin tensor have the same dtype")
    _check(q.dtype == k.dtype and q.device == k.device, "q and k must have the same dtype and device")
    _check(q.size(0) == k.size(0) and q.size(1) == k.size(1) and q.size(3) == k.size(3),
           "q and k must agree in sequence length, batch size and head dimension")
    _check(cos.dtype == torch.float32 or cos.dtype == q.dtype,
           f"{name}: cos/sin must be float32 or have the dtype of the input")
    _hp.require_gpu(cos, name)
    _hp.require_gpu(sin, name)
    c = cos.contiguous()
    sn = sin.contiguous()
    if out is None:
        q_out = _new_output(q, transpose_output)
        k_out = _new_output(k, transpose_output)
    else:
        # caller-provided results with any strides, e.g. two slices of one buffer
        q_out, k_out = out
        for o, t, what in ((q_out, q, "q"), (k_out, k, "k")):
            _check(o.shape == t.shape and o.dtype == t.dtype and o.device == t.device,
                   f"{name}: the result tensor for {what} must match it in shape, dtype and device")
    s, b, hq, d = q.shape
    with _hp.device_guard(q):
        rc = fn(q_out.data_ptr(), k_out.data_ptr(), q.data_ptr(), k.data_ptr(), c.data_ptr(), sn.data_ptr(), s, b, hq,
                k.size(2), d, c.size(3), _hp.strides4(q), _hp.strides4(k), _hp.strides4(q_out), _hp.strides4(k_out),
                _hp.dtype_code(q, name), _hp.dtype_code(c, name), _hp.stream_of(q))
    _hp.check(rc, name)
    return q_out, k_out


def forward_cached_qk(q, k, cos, sin, transpose_output, out=None):
    """(not in the reference module) ``forward_cached`` for q and k in one launch; k may have fewer heads.
    ``out``: optional ``(q_result, k_result)`` tensors to write into (any strides) instead of new ones."""
    return _run_cached_qk("fused_rotary_positional_embedding.forward_cached_qk", _hp.lib().nhp_rope_cached_qk_fwd, q, k,
                          cos, sin, transpose_output, out)


def backward_cached_qk(grad_q, grad_k, cos, sin, transpose_output, out=None):
    """(not in the reference module) ``backward_cached`` for the gradients of q and k in one launch.
    ``out``: optional ``(q_result, k_result)`` tensors to write into (any strides) instead of new ones."""
    return _run_cached_qk("fused_rotary_positional_embedding.backward_cached_qk", _hp.lib().nhp_rope_cached_qk_bwd,
                          grad_q, grad_k, cos, sin, transpose_output, out)


def _run_freqs_qk(name, fn, q, k, freqs, transpose_output):
    for t, what in ((q, "q"), (k, "k")):
        _check(t.dim() == 4, "expected 4D tensor")
        _check(t.size(0) == freqs.size(0), f"expected {what} and freqs tensor have the same sequence length")
        _check(t.size(3) >= freqs.size(3),
               f"expected the last dim of the {what} tensor equals or is greater than the freqs tensor")
        _check(t.dtype in _FLOATS, f"{name}: unsupported dtype {t.dtype}")
        _hp.require_gpu(t, name)
    _check(freqs.dim() == 4, "expected 4D tensor")
    _check(freqs.size(1) == 1 and freqs.size(2) == 1, "expected the second and third dims of the freqs tensor equal 1")
    _check(freqs.dtype == torch.float32, "Dtype of the freqs tensor must be float")
    _check(q.dtype == k.dtype and q.device == k.device, "q and k must have the same dtype and device")
    _check(q.size(0) == k.size(0) and q.size(1) == k.size(1) and q.size(3) == k.size(3),
           "q and k must agree in sequence length, batch size and head dimension")
    _hp.require_gpu(freqs, name)
    f = freqs.contiguous()
    q_out = _new_output(q, transpose_output)
    k_out = _new_output(k, transpose_output)
    s, b, hq, d = q.shape
    with _hp.device_guard(q):
        rc = fn(q_out.data_ptr(), k_out.data_ptr(), q.data_ptr(), k.data_ptr(), f.data_ptr(), s, b, hq, k.size(2), d,
                f.size(3), _hp.strides4(q), _hp.strides4(k), _hp.strides4(q_out), _hp.strides4(k_out),
                _hp.dtype_code(q, name), _hp.stream_of(q))
    _hp.check(rc, name)
    return q_out, k_out


def forward_qk(q, k, freqs, transpose_output):
    """(not in the reference module) ``forward`` for q and k in one launch; k may have fewer heads."""
    return _run_freqs_qk("fused_rotary_positional_embedding.forward_qk", _hp.lib().nhp_rope_freqs_qk_fwd, q, k, freqs,
                         transpose_output)


def backward_qk(grad_q, grad_k, freqs, transpose_output):
    """(not in the reference module) ``backward`` for the gradients of q and k in one launch."""
    return _run_freqs_qk("fused_rotary_positional_embedding.backward_qk", _hp.lib().nhp_rope_freqs_qk_bwd, grad_q, grad_k,
                         freqs, transpose_output)
