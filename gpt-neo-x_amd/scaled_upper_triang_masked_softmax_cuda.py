"""Extension-module surface of the causal fused softmax.

Same functions as the reference's pybind module
(megatron/fused_kernels/scaled_upper_triang_masked_softmax.cpp:62-70), served
by libneox_hotpath.so. Launches are asynchronous on the current stream.
"""
import torch

from megatron.fused_kernels import _hotpath as _hp

_HALF = (torch.float16, torch.bfloat16)


def _key_lengths_arg(key_lengths, attn_batches, heads, who):
    """(tensor kept alive, pointer, heads per batch entry) for an integer [batch] tensor of key counts."""
    if key_lengths is None:
        return None, None, heads
    if key_lengths.dim() != 1 or key_lengths.numel() == 0 or key_lengths.is_floating_point():
        raise RuntimeError("key_lengths must be a non-empty 1-D integer tensor")
    _hp.require_gpu(key_lengths, who)
    batch = key_lengths.numel()
    if attn_batches % batch != 0 or (heads is not None and attn_batches != batch * heads):
        raise RuntimeError("attn_batches must equal len(key_lengths) * heads")
    lengths = key_lengths.to(torch.int32).contiguous()
    return lengths, lengths.data_ptr(), attn_batches // batch


def _per_head_args(x, alibi_slopes, bias, key_lengths, who):
    """Pointers of the optional per-head operands of the forward kernels, the tensors that keep them alive,
    and the number of heads per batch entry they imply (None without any of them)."""
    keep = []
    slopes_ptr, heads = None, None
    if alibi_slopes is not None:
        if alibi_slopes.dtype != torch.float32 or alibi_slopes.dim() != 1:
            raise RuntimeError("alibi_slopes must be a 1-D float32 tensor")
        _hp.require_gpu(alibi_slopes, who)
        alibi_slopes = alibi_slopes.contiguous()
        keep.append(alibi_slopes)
        slopes_ptr, heads = alibi_slopes.data_ptr(), alibi_slopes.numel()
        if heads == 0 or x.size(0) % heads != 0:
            raise RuntimeError("attn_batches must be a multiple of the number of AliBi slopes")
    bias_ptr = None
    if bias is not None:
        if bias.dim() == 4 and bias.size(0) == 1:
            bias = bias[0]
        if bias.dim() != 3 or bias.size(1) != x.size(1) or bias.size(2) != x.size(2) or bias.dtype != x.dtype:
            raise RuntimeError("bias must be [heads, seq_len, seq_len] in the dtype of the input")
        _hp.require_gpu(bias, who)
        if alibi_slopes is not None and bias.size(0) != heads:
            raise RuntimeError("bias and alibi_slopes must have the same number of heads")
        bias = bias.contiguous()
        keep.append(bias)
        bias_ptr, heads = bias.data_ptr(), bias.size(0)
        if heads == 0 or x.size(0) % heads != 0:
            raise RuntimeError("attn_batches must be a multiple of the number of bias heads")
    lengths, lengths_ptr, heads = _key_lengths_arg(key_lengths, x.size(0), heads, who)
    keep.append(lengths)
    return keep, slopes_ptr, bias_ptr, lengths_ptr, heads


def _zero_block(zero_block):
    zero_block = int(zero_block or 0)
    if zero_block and (zero_block < 8 or zero_block & (zero_block - 1)):
        raise RuntimeError("zero_block must be 0 or a power of two of at least 8")
    return zero_block


def forward(input, scale_factor, window=None, alibi_slopes=None, bias=None, key_lengths=None, zero_block=0, *,
            narrow_scale=False):
    """softmax(scale * input) under an upper-triangular mask.

    input: [attn_batches, seq_len, seq_len] fp16/bf16 on the GPU. Returns a new
    tensor of the same shape and dtype (requires_grad False). Checks follow
    scaled_upper_triang_masked_softmax.cpp:31-39; seq_len is not limited to 2048.

    Four optional arguments go beyond the reference function:
    window: sliding-window width; row q attends to keys q-window..q only.
    alibi_slopes: fp32 tensor [heads] on the GPU (attn_batches % heads == 0);
        the AliBi bias -(q-k)*slope is added to the scores in the storage dtype
        before the softmax, as `scores + alibi_matrix` would.
    bias: [heads, seq_len, seq_len] tensor of the input's dtype (attn_batches %
        heads == 0), added to the scores in the storage dtype first, as
        `scores += bias` would (e.g. a relative-position bias shared by the batch).
    key_lengths: integer tensor [batch] on the GPU, input being [batch * heads, s, s]:
        keys at or beyond a batch entry's length are padding and get probability 0
        (a row without any key left is 1/seq_len in every column, as on the torch branch).
    zero_block: for a caller that reads the result in square blocks of this many rows and columns
        and skips the blocks without a visible (query, key) pair: row q is only written from the
        start of the block of the first key that the first row of its block sees to the end of the
        block of the diagonal; the rest of the returned tensor is uninitialised. 0: every row whole.
    narrow_scale (keyword only): round ``scale_factor`` to the input's dtype before use, as the reference's
        CUDA forward does (scaled_upper_triang_masked_softmax.h:368 takes ``const input_t scale``): results
        then follow the reference's fused kernel; by default the fp32 value is used, as in the reference's
        backward and torch branch. 1/sqrt(128) narrows to 0.08837890625 in fp16 and bf16 (-1.07e-4 relative).
    """
    if input.dim() != 3:
        raise RuntimeError("expected 3D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if input.size(1) != input.size(2):
        raise RuntimeError("expected a square [attn_batches, seq_len, seq_len] tensor")
    _hp.require_gpu(input, "scaled_upper_triang_masked_softmax_cuda.forward")
    x = input.contiguous()
    y = torch.empty_like(x)
    keep, slopes_ptr, bias_ptr, lengths_ptr, heads = _per_head_args(
        x, alibi_slopes, bias, key_lengths, "scaled_upper_triang_masked_softmax_cuda.forward")
    with _hp.device_guard(x):
        rc = _hp.lib().nhp_causal_softmax_blocks_fwd(
            y.data_ptr(), x.data_ptr(), _hp.forward_scale(scale_factor, x, narrow_scale), x.size(0), x.size(1),
            -1 if window is None else int(window), _zero_block(zero_block), slopes_ptr, bias_ptr, lengths_ptr, heads or 1,
            _hp.dtype_code(x, "forward"), _hp.stream_of(x))
    _hp.check(rc, "scaled_upper_triang_masked_softmax_cuda.forward")
    return y


def backward(output_grads, softmax_results, scale_factor, window=None, key_lengths=None, zero_block=0):
    """Gradient w.r.t. the input of ``forward`` (pass the same ``window`` and ``key_lengths``;
    AliBi and the bias tensor need nothing here; ``zero_block`` as in ``forward``: only that part
    of every row is read and written).

    Works in place: the result is written into (the contiguous version of)
    ``output_grads`` and that tensor is returned, as in
    scaled_upper_triang_masked_softmax_cuda.cu:61-90.
    """
    if output_grads.dim() != 3 or softmax_results.dim() != 3:
        raise RuntimeError("expected 3D tensor")
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.shape != softmax_results.shape or output_grads.dtype != softmax_results.dtype:
        raise RuntimeError("output_grads and softmax_results must have the same shape and dtype")
    if output_grads.size(1) != output_grads.size(2):
        raise RuntimeError("expected a square [attn_batches, seq_len, seq_len] tensor")
    _hp.require_gpu(output_grads, "scaled_upper_triang_masked_softmax_cuda.backward")
    _hp.require_gpu(softmax_results, "scaled_upper_triang_masked_softmax_cuda.backward")
    g = output_grads.detach().contiguous()
    y = softmax_results.detach().contiguous()
    lengths, lengths_ptr, heads = _key_lengths_arg(key_lengths, g.size(0), None,
                                                   "scaled_upper_triang_masked_softmax_cuda.backward")
    with _hp.device_guard(g):
        rc = _hp.lib().nhp_causal_softmax_blocks_bwd(
            g.data_ptr(), g.data_ptr(), y.data_ptr(), float(scale_factor), g.size(0), g.size(1),
            -1 if window is None else int(window), _zero_block(zero_block), lengths_ptr, heads or 1,
            _hp.dtype_code(g, "backward"),
            _hp.stream_of(g))
    _hp.check(rc, "scaled_upper_triang_masked_softmax_cuda.backward")
    return g


def forward_dropout(input, scale_factor, p, seed, window=None, zero_block=0, alibi_slopes=None, bias=None,
                    key_lengths=None, *, narrow_scale=False):
    """``forward`` and attention dropout in one kernel: returns ``(dropped, probabilities)``.

    ``dropped = keep * probabilities / (1 - p)`` with the library's counter-based keep mask for
    ``seed`` (see ``nhp_causal_softmax_dropout_fwd``); ``probabilities`` is what ``forward`` returns
    and what ``backward_dropout`` needs. ``alibi_slopes``, ``bias``, ``key_lengths`` and ``narrow_scale`` as in ``forward``.
    Not part of the reference's extension module."""
    who = "scaled_upper_triang_masked_softmax_cuda.forward_dropout"
    if input.dim() != 3:
        raise RuntimeError("expected 3D tensor")
    if input.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if input.size(1) != input.size(2):
        raise RuntimeError("expected a square [attn_batches, seq_len, seq_len] tensor")
    _hp.require_gpu(input, who)
    x = input.contiguous()
    y = torch.empty_like(x)
    dropped = torch.empty_like(x)
    keep, slopes_ptr, bias_ptr, lengths_ptr, heads = _per_head_args(x, alibi_slopes, bias, key_lengths, who)
    with _hp.device_guard(x):
        rc = _hp.lib().nhp_causal_softmax_ex_dropout_fwd(
            dropped.data_ptr(), y.data_ptr(), x.data_ptr(), _hp.forward_scale(scale_factor, x, narrow_scale), x.size(0),
            x.size(1), -1 if window is None else int(window), _zero_block(zero_block), slopes_ptr, bias_ptr, lengths_ptr,
            heads or 1, float(p), int(seed), 0, _hp.dtype_code(x, "forward_dropout"), _hp.stream_of(x))
    _hp.check(rc, who)
    del keep
    return dropped, y


def backward_dropout(output_grads, softmax_results, scale_factor, p, seed, window=None, zero_block=0, key_lengths=None):
    """Gradient of ``forward_dropout`` with respect to its input, given the gradient of ``dropped``
    (pass the same ``window``, ``zero_block`` and ``key_lengths``); in place on ``output_grads`` like ``backward``."""
    who = "scaled_upper_triang_masked_softmax_cuda.backward_dropout"
    if output_grads.dim() != 3 or softmax_results.dim() != 3:
        raise RuntimeError("expected 3D tensor")
    if output_grads.dtype not in _HALF or softmax_results.dtype not in _HALF:
        raise RuntimeError("Only fp16 and bf16 are supported")
    if output_grads.shape != softmax_results.shape or output_grads.dtype != softmax_results.dtype:
        raise RuntimeError("output_grads and softmax_results must have the same shape and dtype")
    _hp.require_gpu(output_grads, who)
    _hp.require_gpu(softmax_results, who)
    g = output_grads.detach().contiguous()
    y = softmax_results.detach().contiguous()
    lengths, lengths_ptr, heads = _key_lengths_arg(key_lengths, g.size(0), None, who)
    with _hp.device_guard(g):
        rc = _hp.lib().nhp_causal_softmax_ex_dropout_bwd(
            g.data_ptr(), g.data_ptr(), y.data_ptr(), float(scale_factor), g.size(0), g.size(1),
            -1 if window is None else int(window), _zero_block(zero_block), lengths_ptr, heads or 1, float(p),
            int(seed), 0, _hp.dtype_code(g, "backward_dropout"), _hp.stream_of(g))
    _hp.check(rc, who)
    del lengths
    return g
