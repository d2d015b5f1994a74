"""Extension-module surface of the padding-masked fused softmax.

Same functions as the reference's pybind module
(megatron/fused_kernels/scaled_masked_softmax.cpp:70-83), served by
libneox_hotpath.so. Launches are asynchronous on the current stream.
"""
import torch

from megatron.fused_kernels import _hotpath as _hp

_HALF = (torch.float16, torch.bfloat16)


def _checked_forward_args(input, mask, name):
    if input.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if mask.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if mask.element_size() != 1:
        raise RuntimeError("mask must have one byte per element (bool or uint8)")
    b, np_, sq, sk = input.shape
    if not sq > 1:
        raise RuntimeError("query_seq_len > 1 INTERNAL ASSERT FAILED")
    if mask.size(0) != 1 and mask.size(0) != b:
        raise RuntimeError("pad_batches == 1 || pad_batches == batches INTERNAL ASSERT FAILED")
    if mask.size(1) != 1 or mask.size(2) != sq or mask.size(3) != sk:
        raise RuntimeError("mask must have shape [pad_batches, 1, query_seq_len, key_seq_len]")
    _hp.require_gpu(input, name)
    _hp.require_gpu(mask, name)
    return input.contiguous(), mask.contiguous()


def _extras(x, alibi_slopes, bias, key_lengths, name):
    """Pointers (and the tensors that keep them alive) of the optional operands of ``forward``."""
    b, np_, sq, sk = x.shape
    keep = []
    slopes_ptr = bias_ptr = lengths_ptr = None
    if alibi_slopes is not None:
        if alibi_slopes.dtype != torch.float32 or alibi_slopes.dim() != 1 or alibi_slopes.numel() != np_:
            raise RuntimeError("alibi_slopes must be a float32 tensor with one slope per head")
        if sq != sk:
            raise RuntimeError("the AliBi bias needs query_seq_len == key_seq_len")
        _hp.require_gpu(alibi_slopes, name)
        keep.append(alibi_slopes.contiguous())
        slopes_ptr = keep[-1].data_ptr()
    if bias is not None:
        if bias.dim() == 4 and bias.size(0) == 1:
            bias = bias[0]
        if bias.shape != (np_, sq, sk) or bias.dtype != x.dtype:
            raise RuntimeError("bias must be [heads, query_seq_len, key_seq_len] in the dtype of the input")
        _hp.require_gpu(bias, name)
        keep.append(bias.contiguous())
        bias_ptr = keep[-1].data_ptr()
    if key_lengths is not None:
        if key_lengths.dim() != 1 or key_lengths.numel() != b or key_lengths.is_floating_point():
            raise RuntimeError("key_lengths must be an integer tensor with one entry per batch entry")
        _hp.require_gpu(key_lengths, name)
        keep.append(key_lengths.to(torch.int32).contiguous())
        lengths_ptr = keep[-1].data_ptr()
    return keep, slopes_ptr, bias_ptr, lengths_ptr


def forward(input, mask, scale_factor, alibi_slopes=None, bias=None, key_lengths=None, *, narrow_scale=False):
    """softmax(where(mask == 1, -10000, scale * input)) over the last dim.

    input: [b, np, sq, sk] fp16/bf16; mask: [1 or b, 1, sq, sk], one byte per
    element (bool or uint8). Checks follow scaled_masked_softmax.cpp:33-42 and
    scaled_masked_softmax_cuda.cu:46-51; sk is not limited to 2048.

    Three optional arguments go beyond the reference function; each stands for a pass over the scores
    (or the mask) that the caller otherwise makes first (megatron/model/transformer.py:580-588):
    alibi_slopes: fp32 [np] on the GPU, needs sq == sk: ``scores + alibi_matrix`` in the storage dtype;
    bias: [np, sq, sk] (or [1, np, sq, sk]) in the input's dtype: ``scores += bias`` in the storage dtype;
    key_lengths: integer [b] on the GPU: keys at or beyond a batch entry's length count as masked.
    narrow_scale (keyword only): round ``scale_factor`` to the input's dtype before use, as the reference's CUDA
    forward does (scaled_masked_softmax.h:358 takes ``const input_t scale``); by default the fp32 value is used,
    as in the reference's backward and torch branch.
    """
    name = "scaled_masked_softmax_cuda.forward"
    x, m = _checked_forward_args(input, mask, name)
    b, np_, sq, sk = x.shape
    keep, slopes_ptr, bias_ptr, lengths_ptr = _extras(x, alibi_slopes, bias, key_lengths, name)
    y = torch.empty_like(x)
    with _hp.device_guard(x):
        rc = _hp.lib().nhp_masked_softmax_ex_fwd(
            y.data_ptr(), x.data_ptr(), m.data_ptr(), _hp.forward_scale(scale_factor, x, narrow_scale), b, np_, sq, sk,
            m.size(0), slopes_ptr, bias_ptr, lengths_ptr, _hp.dtype_code(x, "forward"), _hp.stream_of(x))
    _hp.check(rc, name)
    del keep
    return y


def backward(output_grads, softmax_results, scale_factor):
    """Gradient w.r.t. the input of ``forward`` (no mask is applied). Works in
    place on (the contiguous version of) ``output_grads`` and returns it, as in
    scaled_masked_softmax_cuda.cu:78-108."""
    if output_grads.dim() != 4 or softmax_results.dim() != 4:
        raise RuntimeError("expected 3D tensor")  # wording of the reference's check on 4-D inputs
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.shape != softmax_results.shape or output_grads.dtype != softmax_results.dtype:
        raise RuntimeError("output_grads and softmax_results must have the same shape and dtype")
    _hp.require_gpu(output_grads, "scaled_masked_softmax_cuda.backward")
    _hp.require_gpu(softmax_results, "scaled_masked_softmax_cuda.backward")
    g = output_grads.detach().contiguous()
    y = softmax_results.detach().contiguous()
    sk = g.size(3)
    rows = g.numel() // sk if sk else 0
    with _hp.device_guard(g):
        rc = _hp.lib().nhp_masked_softmax_bwd(
            g.data_ptr(), g.data_ptr(), y.data_ptr(), float(scale_factor), rows, sk,
            _hp.dtype_code(g, "backward"), _hp.stream_of(g))
    _hp.check(rc, "scaled_masked_softmax_cuda.backward")
    return g


def _check_prob(p, name):
    if not 0.0 <= float(p) < 1.0:
        raise RuntimeError(f"{name}: dropout probability has to be in [0, 1), got {p}")


def forward_dropout(input, mask, scale_factor, p, seed, alibi_slopes=None, bias=None, key_lengths=None, *,
                    narrow_scale=False):
    """(not in the reference module) ``forward`` and attention dropout in one kernel: returns
    ``(dropped, probs)`` with ``dropped = keep ? probs / (1 - p) : 0``; the keep mask is generated from
    ``seed`` over the flat element index and is regenerated by ``backward_dropout``."""
    name = "scaled_masked_softmax_cuda.forward_dropout"
    _check_prob(p, name)
    x, m = _checked_forward_args(input, mask, name)
    b, np_, sq, sk = x.shape
    keep, slopes_ptr, bias_ptr, lengths_ptr = _extras(x, alibi_slopes, bias, key_lengths, name)
    y = torch.empty_like(x)
    dropped = torch.empty_like(x)
    with _hp.device_guard(x):
        rc = _hp.lib().nhp_masked_softmax_ex_dropout_fwd(
            dropped.data_ptr(), y.data_ptr(), x.data_ptr(), m.data_ptr(), _hp.forward_scale(scale_factor, x, narrow_scale),
            b, np_, sq, sk, m.size(0), slopes_ptr, bias_ptr, lengths_ptr, float(p), int(seed), 0, _hp.dtype_code(x, name), _hp.stream_of(x))
    _hp.check(rc, name)
    del keep
    return dropped, y


def backward_dropout(output_grads, softmax_results, scale_factor, p, seed):
    """(not in the reference module) gradient of ``forward_dropout`` with respect to its input, given the
    gradient of ``dropped``; in place on (the contiguous version of) ``output_grads`` like ``backward``."""
    name = "scaled_masked_softmax_cuda.backward_dropout"
    _check_prob(p, name)
    if output_grads.dim() != 4 or softmax_results.dim() != 4:
        raise RuntimeError("expected 4D tensor")
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.shape != softmax_results.shape or output_grads.dtype != softmax_results.dtype:
        raise RuntimeError("output_grads and softmax_results must have the same shape and dtype")
    _hp.require_gpu(output_grads, name)
    _hp.require_gpu(softmax_results, name)
    g = output_grads.detach().contiguous()
    y = softmax_results.detach().contiguous()
    sk = g.size(3)
    rows = g.numel() // sk if sk else 0
    with _hp.device_guard(g):
        rc = _hp.lib().nhp_masked_softmax_dropout_bwd(
            g.data_ptr(), g.data_ptr(), y.data_ptr(), float(scale_factor), rows, sk, float(p), int(seed), 0,
            _hp.dtype_code(g, name), _hp.stream_of(g))
    _hp.check(rc, name)
    return g


def get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads):
    """Rows per 128-thread block of the reference launch geometry on a 64-wide
    wavefront (scaled_masked_softmax.h:338-352); used by the fusion gate only."""
    rc = _hp.lib().nhp_softmax_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads)
    if rc < 0:
        _hp.check(rc, "scaled_masked_softmax_cuda.get_batch_per_block")
    return rc
