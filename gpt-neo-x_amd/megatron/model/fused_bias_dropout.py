"""bias + dropout + residual add on MI355X.

Surface of GPT-NeoX's ``megatron/model/fused_bias_dropout.py``:
``bias_dropout_add`` (:28-35), ``get_bias_dropout_add`` (:38-42),
``bias_dropout_add_fused_train`` (:45-50), ``bias_dropout_add_fused_inference``
(:53-58). The whole expression ``residual + dropout(x + bias)`` is one gfx950
kernel, evaluated in fp32 and rounded once. With dropout active the keep mask
comes from the library's own counter-based generator (Philox4x32-10 over the
flat element index, seeded per call from the device's CUDA generator, see
``dropout_rng``, so ``torch.manual_seed`` makes runs repeatable); it is
regenerated in the backward instead of being stored.

Parity of the keep mask is unpinned against the reference by construction: WHICH
elements are dropped for a given seed is this library's definition, not that of
``torch.nn.functional.dropout`` (which the reference calls and which draws its
mask from torch's generator stream in its own order). Everything else is pinned:
the generator against the published Philox4x32-10 known answers, the keep rate,
and ``keep ? (x + bias) / (1 - p) : 0`` plus the residual bit for bit given the mask.
With dropout off (``training=False`` or ``prob=0``, the setting of every
configuration the reference ships) results do not depend on any of this.
"""
from typing import Optional

import torch
from torch import Tensor

from ..fused_kernels import _hotpath as _hp


def _bias_vector(bias, x, what):
    """The bias as a contiguous ``[cols]`` vector, and whether it came expanded to the shape of ``x``
    (the reference's call sites pass ``bias.expand_as(residual)``, megatron/model/transformer.py:1229,1271)."""
    if bias is None:
        return None, False
    cols = x.size(-1)
    _hp.require_gpu(bias, what)
    if bias.dtype != x.dtype:
        raise RuntimeError(f"{what}: bias must hold one value per feature, in the dtype of x")
    if bias.numel() == cols:
        return bias.contiguous().view(-1), False
    if bias.shape == x.shape and all(st == 0 or sz == 1 for st, sz in zip(bias.stride()[:-1], bias.shape[:-1])):
        row = bias.detach().as_strided((cols,), (bias.stride(-1),), bias.storage_offset())
        return row.contiguous(), True
    raise RuntimeError(f"{what}: bias must hold one value per feature (a vector, or one expanded to the shape of x)")


def _prepare(x, bias, residual, what):
    _hp.require_gpu(x, what)
    cols = x.size(-1)
    src = x.contiguous()
    b, expanded = _bias_vector(bias, x, what)
    res = None
    if residual is not None:
        if residual.shape != x.shape or residual.dtype != x.dtype:
            raise RuntimeError(f"{what}: residual and x must have the same shape and dtype")
        _hp.require_gpu(residual, what)
        res = residual.contiguous()
    return src, b, res, src.numel() // max(cols, 1), cols, expanded


def _bias_grad(per_element, bias_shape, expanded):
    """Gradient for the bias argument: of an expanded bias every element has its own gradient (autograd
    sums them when it undoes the expansion); for a vector the rows are summed here."""
    if expanded:
        return per_element
    return _column_sum(per_element).view(bias_shape)


def _column_sum(t):
    """Sum over all but the last dimension, fp32 accumulation in a fixed order, one rounding."""
    what = "bias_dropout_add backward"
    cols = t.size(-1)
    src = t.contiguous()
    rows = src.numel() // max(cols, 1)
    out = torch.zeros(cols, dtype=src.dtype, device=src.device) if rows == 0 else \
        torch.empty(cols, dtype=src.dtype, device=src.device)
    code = _hp.dtype_code(src, what)
    nbytes = _hp.lib().nhp_column_sum_workspace_bytes(rows, cols, code)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=src.device) if nbytes else None
    with _hp.device_guard(src):
        rc = _hp.lib().nhp_column_sum(out.data_ptr(), src.data_ptr(), None if ws is None else ws.data_ptr(), rows, cols,
                                      code, _hp.stream_of(src))
    _hp.check(rc, what)
    return out


class _BiasAddResidual(torch.autograd.Function):
    """``residual + (x + bias)``: the gradient passes through unchanged to ``x`` and
    ``residual`` and is summed over rows for ``bias``."""

    @staticmethod
    def forward(ctx, x, bias, residual):
        what = "bias_dropout_add"
        src, b, res, rows, cols, expanded = _prepare(x, bias, residual, what)
        out = torch.empty_like(src)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_bias_add_residual(out.data_ptr(), src.data_ptr(), None if b is None else b.data_ptr(),
                                                 None if res is None else res.data_ptr(), rows, cols,
                                                 _hp.dtype_code(src, what), _hp.stream_of(src))
        _hp.check(rc, what)
        ctx.conf = (None if bias is None else bias.shape, expanded)
        return out

    @staticmethod
    def backward(ctx, grad):
        bias_shape, expanded = ctx.conf
        gb = None
        if bias_shape is not None and ctx.needs_input_grad[1]:
            gb = _bias_grad(grad, bias_shape, expanded)
        return grad, gb, grad if ctx.needs_input_grad[2] else None


class _BiasAddResidualPair(torch.autograd.Function):
    """``residual + ((x1 + bias1) + (x2 + bias2))`` in one pass, rounded as the three separate additions round.
    The gradient passes through unchanged to ``x1``, ``x2`` and ``residual``; the two biases share one sum of it
    over the rows."""

    @staticmethod
    def forward(ctx, x1, bias1, x2, bias2, residual):
        what = "bias_add_residual_pair"
        a, b1, res, rows, cols, exp1 = _prepare(x1, bias1, residual, what)
        if res is None:
            raise RuntimeError(f"{what}: a residual is required")
        if x2.shape != x1.shape or x2.dtype != x1.dtype:
            raise RuntimeError(f"{what}: x1 and x2 must have the same shape and dtype")
        _hp.require_gpu(x2, what)
        b2, exp2 = _bias_vector(bias2, x2, what)
        c = x2.contiguous()
        out = torch.empty_like(a)
        with _hp.device_guard(a):
            rc = _hp.lib().nhp_bias_add_residual_pair(
                out.data_ptr(), a.data_ptr(), None if b1 is None else b1.data_ptr(), c.data_ptr(),
                None if b2 is None else b2.data_ptr(), res.data_ptr(), rows, cols, _hp.dtype_code(a, what),
                _hp.stream_of(a))
        _hp.check(rc, what)
        ctx.conf = (None if bias1 is None else bias1.shape, exp1, None if bias2 is None else bias2.shape, exp2)
        return out

    @staticmethod
    def backward(ctx, grad):
        shape1, exp1, shape2, exp2 = ctx.conf
        need1 = shape1 is not None and ctx.needs_input_grad[1]
        need2 = shape2 is not None and ctx.needs_input_grad[3]
        summed = _column_sum(grad) if (need1 and not exp1) or (need2 and not exp2) else None
        g1 = (grad if exp1 else summed.view(shape1)) if need1 else None
        g2 = (grad if exp2 else summed.view(shape2)) if need2 else None
        return grad, g1, grad, g2, grad if ctx.needs_input_grad[4] else None


def bias_add_residual_pair(x1: Tensor, bias1: Optional[Tensor], x2: Tensor, bias2: Optional[Tensor],
                           residual: Tensor) -> Tensor:
    """``residual + ((x1 + bias1) + (x2 + bias2))``: how the parallel-residual layer combines the outputs of its
    attention and MLP branches (three ``bias_dropout_add`` calls in ParallelTransformerLayer.forward,
    megatron/model/transformer.py:1229-1250) when dropout is off, in one kernel and with the reference's
    roundings."""
    return _BiasAddResidualPair.apply(x1, bias1, x2, bias2, residual)


class _BiasDropoutAdd(torch.autograd.Function):
    """``residual + dropout(x + bias)`` with the mask regenerated from (seed, prob) in the backward."""

    @staticmethod
    def forward(ctx, x, bias, residual, prob, seed):
        what = "bias_dropout_add"
        src, b, res, rows, cols, expanded = _prepare(x, bias, residual, what)
        out = torch.empty_like(src)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_bias_dropout_add(out.data_ptr(), src.data_ptr(), None if b is None else b.data_ptr(),
                                                None if res is None else res.data_ptr(), rows, cols, float(prob), seed,
                                                0, _hp.dtype_code(src, what), _hp.stream_of(src))
        _hp.check(rc, what)
        ctx.conf = (float(prob), seed, None if bias is None else bias.shape, expanded)
        return out

    @staticmethod
    def backward(ctx, grad):
        what = "bias_dropout_add backward"
        prob, seed, bias_shape, expanded = ctx.conf
        g = grad.contiguous()
        cols = g.size(-1)
        rows = g.numel() // max(cols, 1)
        dx = torch.empty_like(g)
        with _hp.device_guard(g):
            rc = _hp.lib().nhp_dropout_bwd(dx.data_ptr(), g.data_ptr(), rows, cols, prob, seed, 0,
                                           _hp.dtype_code(g, what), _hp.stream_of(g))
        _hp.check(rc, what)
        gb = None
        if bias_shape is not None and ctx.needs_input_grad[1]:
            gb = _bias_grad(dx, bias_shape, expanded)
        return dx, gb, grad if ctx.needs_input_grad[2] else None, None, None


def _fresh_seed(device):
    # from the device's CUDA generator, read on the host: follows torch.manual_seed, no synchronisation
    from . import dropout_rng

    return dropout_rng.next_seed(device)


def bias_dropout_add(x: Tensor, bias: Tensor, residual: Optional[Tensor], prob: float, training: bool) -> Tensor:
    if training and prob > 0.0:
        if not prob < 1.0:
            raise ValueError(f"dropout probability has to be between 0 and 1, but got {prob}")
        return _BiasDropoutAdd.apply(x, bias, residual, prob, _fresh_seed(x.device))
    return _BiasAddResidual.apply(x, bias, residual)


def get_bias_dropout_add(training):
    def _bias_dropout_add(x, bias, residual, prob):
        return bias_dropout_add(x, bias, residual, prob, training)

    return _bias_dropout_add


def bias_dropout_add_fused_train(x: Tensor, bias: Tensor, residual: Optional[Tensor], prob: float) -> Tensor:
    return bias_dropout_add(x, bias, residual, prob, True)


def bias_dropout_add_fused_inference(x: Tensor, bias: Tensor, residual: Optional[Tensor], prob: float) -> Tensor:
    return bias_dropout_add(x, bias, residual, prob, False)
