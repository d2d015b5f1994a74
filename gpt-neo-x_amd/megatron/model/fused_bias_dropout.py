"""bias + dropout + residual add on MI355X.

Surface of GPT-NeoX's ``megatron/model/fused_bias_dropout.py``:
``bias_dropout_add`` (:28-35), ``get_bias_dropout_add`` (:38-42),
``bias_dropout_add_fused_train`` (:45-50), ``bias_dropout_add_fused_inference``
(:53-58). The whole expression ``residual + dropout(x + bias)`` is one gfx950
kernel, evaluated in fp32 and rounded once. With dropout active the keep mask
comes from the library's own counter-based generator (Philox4x32-10, seeded
per call from torch's CPU generator, so ``torch.manual_seed`` makes runs
repeatable); it is regenerated in the backward instead of being stored. Which
elements are dropped therefore differs from what torch's dropout would pick.
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


def _fresh_seed():
    # from torch's CPU generator: no device synchronisation, repeatable under torch.manual_seed
    return int(torch.empty((), dtype=torch.int64).random_().item())


def bias_dropout_add(x: Tensor, bias: Tensor, residual: Optional[Tensor], prob: float, training: bool) -> Tensor:
    if training and prob > 0.0:
        if not prob < 1.0:
            raise ValueError(f"dropout probability has to be between 0 and 1, but got {prob}")
        return _BiasDropoutAdd.apply(x, bias, residual, prob, _fresh_seed())
    return _BiasAddResidual.apply(x, bias, residual)


def get_bias_dropout_add(training):
    def _bias_dropout_add(x, bias, residual, prob):
        return bias_dropout_add(x, bias, residual, prob, training)

    return _bias_dropout_add


def bias_dropout_add_fused_train(x: Tensor, bias: Tensor, residual: Optional[Tensor], prob: float) -> Tensor:
    return bias_dropout_add(x, bias, residual, prob, True)


def bias_dropout_add_fused_inference(x: Tensor, bias: Tensor, residual: Optional[Tensor], prob: float) -> Tensor:
    return bias_dropout_add(x, bias, residual, prob, False)
