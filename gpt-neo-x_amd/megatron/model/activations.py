"""bias + GeLU (tanh form) on MI355X.

The fused part of GPT-NeoX's ``megatron/model/activations.py``: ``bias_gelu``
(:79-82), ``bias_gelu_back`` (:88-97), ``GeLUFunction`` (:100-112) and
``bias_gelu_impl`` (:115), with the same arguments. The reference compiles the
two expressions with TorchScript; here each is one hand-written gfx950 kernel
(libneox_hotpath.so), evaluated in fp32 with one rounding to the storage dtype.

One difference, to the caller's advantage: ``GeLUFunction.backward`` returns
the bias gradient already reduced to the bias shape (the column sums are formed
inside the backward kernel) instead of a second full-size tensor that autograd
then has to reduce.
"""
import torch

from ..fused_kernels import _hotpath as _hp


def _as_rows(t, cols, what):
    if t.size(-1) != cols:
        raise RuntimeError(f"{what}: last dimension {t.size(-1)} does not match the bias ({cols})")
    return t.contiguous()


def _check_bias(bias, y, what):
    if bias is None:
        return None
    if bias.dim() != 1 or bias.size(0) != y.size(-1):
        raise RuntimeError(f"{what}: bias must be 1-D with the size of the last dimension of the input")
    if bias.dtype != y.dtype:
        raise RuntimeError(f"{what}: bias and input must have the same dtype")
    _hp.require_gpu(bias, what)
    return bias.contiguous()


def bias_gelu(bias, y):
    """``x = bias + y; x * 0.5 * (1 + tanh(0.79788456 * x * (1 + 0.044715 * x * x)))``."""
    what = "bias_gelu"
    _hp.require_gpu(y, what)
    cols = y.size(-1)
    bias = _check_bias(bias, y, what)
    src = _as_rows(y, cols, what)
    out = torch.empty_like(src)
    rows = src.numel() // max(cols, 1)
    with _hp.device_guard(src):
        rc = _hp.lib().nhp_bias_gelu_fwd(out.data_ptr(), src.data_ptr(), None if bias is None else bias.data_ptr(),
                                         rows, cols, _hp.dtype_code(src, what), _hp.stream_of(src))
    _hp.check(rc, what)
    return out


def _bias_gelu_backward(g, bias, y, want_dbias):
    what = "bias_gelu_back"
    _hp.require_gpu(g, what)
    _hp.require_gpu(y, what)
    if g.shape != y.shape or g.dtype != y.dtype:
        raise RuntimeError(f"{what}: gradient and input must have the same shape and dtype")
    cols = y.size(-1)
    bias = _check_bias(bias, y, what)
    src = _as_rows(y, cols, what)
    grad = g.contiguous()
    dx = torch.empty_like(src)
    rows = src.numel() // max(cols, 1)
    code = _hp.dtype_code(src, what)
    dbias = workspace = None
    if want_dbias and bias is not None:
        dbias = torch.zeros_like(bias) if rows == 0 else torch.empty_like(bias)
        nbytes = _hp.lib().nhp_bias_gelu_bwd_workspace_bytes(rows, cols, code)
        if nbytes:
            workspace = torch.empty(nbytes, dtype=torch.uint8, device=src.device)
    with _hp.device_guard(src):
        rc = _hp.lib().nhp_bias_gelu_bwd(dx.data_ptr(), grad.data_ptr(), src.data_ptr(),
                                         None if bias is None else bias.data_ptr(),
                                         None if dbias is None else dbias.data_ptr(),
                                         None if workspace is None else workspace.data_ptr(),
                                         rows, cols, code, _hp.stream_of(src))
    _hp.check(rc, what)
    return dx, dbias


def bias_gelu_back(g, bias, y):
    """Gradient of ``bias_gelu`` with respect to ``y`` (and, summed over rows, to ``bias``), times ``g``."""
    return _bias_gelu_backward(g, bias, y, False)[0]


class GeLUFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, bias):
        ctx.save_for_backward(input, bias)
        return bias_gelu(bias, input)

    @staticmethod
    def backward(ctx, grad_output):
        input, bias = ctx.saved_tensors
        dx, dbias = _bias_gelu_backward(grad_output, bias, input, ctx.needs_input_grad[1])
        return dx, dbias


bias_gelu_impl = GeLUFunction.apply
