"""Extension-module surface of the padding-masked fused softmax.

Same functions as the reference's pybind module
(megatron/fused_kernels/scaled_masked_softmax.cpp:70-83), served by
libneox_hotpath.so. Launches are asynchronous on the current stream.
"""
import torch

from megatron.fused_kernels import _hotpath as _hp

_HALF = (torch.float16, torch.bfloat16)


def forward(input, mask, scale_factor):
    """softmax(where(mask == 1, -10000, scale * input)) over the last dim.

    input: [b, np, sq, sk] fp16/bf16; mask: [1 or b, 1, sq, sk], one byte per
    element (bool or uint8). Checks follow scaled_masked_softmax.cpp:33-42 and
    scaled_masked_softmax_cuda.cu:46-51; sk is not limited to 2048.
    """
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
    _hp.require_gpu(input, "scaled_masked_softmax_cuda.forward")
    _hp.require_gpu(mask, "scaled_masked_softmax_cuda.forward")
    x = input.contiguous()
    m = mask.contiguous()
    y = torch.empty_like(x)
    with _hp.device_guard(x):
        rc = _hp.lib().nhp_masked_softmax_fwd(
            y.data_ptr(), x.data_ptr(), m.data_ptr(), float(scale_factor), b, np_, sq, sk, m.size(0),
            _hp.dtype_code(x, "forward"), _hp.stream_of(x))
    _hp.check(rc, "scaled_masked_softmax_cuda.forward")
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


def get_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads):
    """Rows per 128-thread block of the reference launch geometry on a 64-wide
    wavefront (scaled_masked_softmax.h:338-352); used by the fusion gate only."""
    rc = _hp.lib().nhp_softmax_batch_per_block(query_seq_len, key_seq_len, batches, attn_heads)
    if rc < 0:
        _hp.check(rc, "scaled_masked_softmax_cuda.get_batch_per_block")
    return rc
