"""bias + GeLU (tanh form) and the gated MLP activations on MI355X.

The fused part of GPT-NeoX's ``megatron/model/activations.py``: ``bias_gelu``
(:79-82), ``bias_gelu_back`` (:88-97), ``GeLUFunction`` (:100-112) and
``bias_gelu_impl`` (:115), with the same arguments. The reference compiles the
two expressions with TorchScript; here each is one hand-written gfx950 kernel
(libneox_hotpath.so), evaluated in fp32 with one rounding to the storage dtype.

``Gated_Activation`` (the class of megatron/model/transformer.py:186-206) with the
activations ``get_activation`` (:30-66) pairs with a gate -- geglu, reglu,
bilinear, swiglu, glu -- is one kernel forward and one backward.

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


# ---------------------------------------------------------------------------
# gated activations
# ---------------------------------------------------------------------------
def swish(x, beta: float = 1.0):
    """``x * sigmoid(beta * x)`` (megatron/model/activations.py:128-130); as a gate only beta = 1 is fused."""
    return x * torch.sigmoid(beta * x)


def _identity(x):
    return x


# what get_activation hands to Gated_Activation for each gated `activation` setting
_GATES = {"swiglu": swish, "geglu": torch.nn.functional.gelu, "reglu": torch.nn.functional.relu,
          "glu": torch.nn.functional.sigmoid, "bilinear": _identity}
_GATE_CODE = {swish: 0, torch.nn.functional.gelu: 1, torch.nn.functional.relu: 2, torch.nn.functional.sigmoid: 3,
              torch.sigmoid: 3, _identity: 4}


def erf_gelu(x):
    """GeLU through erf with the reference's rounded constant, ``x * 0.5 * (erf(x / 1.41421) + 1)``
    (megatron/model/activations.py:117-126)."""
    return x * 0.5 * (torch.erf(x / 1.41421).to(dtype=x.dtype) + torch.ones_like(x).to(dtype=x.dtype))


def mish(x):
    """``x * tanh(softplus(x))`` (megatron/model/activations.py:134-135)."""
    return x * torch.tanh(torch.nn.functional.softplus(x))


# Settings that are one torch call on one tensor in the reference as well (no fused kernel on either side).
_PLAIN = {"relu": torch.nn.functional.relu, "softsign": torch.nn.functional.softsign, "swish": swish, "mish": mish,
          "silu": torch.nn.functional.silu}


def get_activation(neox_args):
    """(activation function, is_gated), as megatron/model/activations.py:27-66. The gated settings and
    ``gelu`` with ``bias_gelu_fusion`` are served by the kernels of this library; the remaining settings
    return the same torch functions as the reference."""
    name = neox_args.activation
    if name in _GATES:
        return _GATES[name], True
    if name == "gelu":
        onnx_safe = getattr(neox_args, "onnx_safe", False)
        fusion = getattr(neox_args, "bias_gelu_fusion", False)
        if onnx_safe and fusion:
            raise ValueError("onnx_safe + bias_gelu_fusion not compatible")
        if onnx_safe:
            return erf_gelu, False
        return (bias_gelu_impl if fusion else torch.nn.functional.gelu), False
    if name in _PLAIN:
        return _PLAIN[name], False
    raise ValueError(f"Activation function {name} not recognized")


class _GatedActivationFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, inp, bias, code):
        what = "Gated_Activation"
        _hp.require_gpu(inp, what)
        if inp.size(-1) % 2:
            raise RuntimeError(f"{what}: the last dimension must be even")
        features = inp.size(-1) // 2
        src = inp.contiguous()
        b = None
        if bias is not None:
            if bias.numel() != 2 * features or bias.dtype != inp.dtype:
                raise RuntimeError(f"{what}: bias must hold 2 * features values in the dtype of the input")
            _hp.require_gpu(bias, what)
            b = bias.contiguous().view(-1)
        out = torch.empty(src.shape[:-1] + (features,), dtype=src.dtype, device=src.device)
        rows = src.numel() // max(2 * features, 1)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_gated_act_fwd(out.data_ptr(), src.data_ptr(), None if b is None else b.data_ptr(), rows,
                                             features, code, _hp.dtype_code(src, what), _hp.stream_of(src))
        _hp.check(rc, what)
        ctx.save_for_backward(src, b)
        ctx.code = code
        ctx.bias_shape = None if bias is None else bias.shape
        return out

    @staticmethod
    def backward(ctx, grad):
        what = "Gated_Activation backward"
        src, b = ctx.saved_tensors
        g = grad.contiguous()
        features = src.size(-1) // 2
        rows = src.numel() // max(2 * features, 1)
        din = torch.empty_like(src)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_gated_act_bwd(din.data_ptr(), g.data_ptr(), src.data_ptr(), None if b is None else b.data_ptr(),
                                             rows, features, ctx.code, _hp.dtype_code(src, what), _hp.stream_of(src))
        _hp.check(rc, what)
        dbias = None
        if b is not None and ctx.needs_input_grad[1]:
            dbias = din.reshape(-1, 2 * features).sum(dim=0).view(ctx.bias_shape)
        return din, dbias, None


class Gated_Activation(torch.nn.Module):
    """``x, gate = x.chunk(2, dim=-1); activation_func(gate + bias_2) * (x + bias_1)``
    (megatron/model/transformer.py:186-206). ``activation_func`` is one of the functions ``get_activation``
    returns for a gated setting (or its name); ``use_swiglu`` is accepted and changes nothing, the fused
    SwiGLU it selects in the reference computes the same expression."""

    def __init__(self, activation_func, use_swiglu=False):
        super().__init__()
        if isinstance(activation_func, str):
            activation_func = _GATES[activation_func]
        if activation_func not in _GATE_CODE:
            raise ValueError("Gated_Activation: activation function not provided by the MI355X kernels")
        self.activation_func = activation_func
        self.use_swiglu = use_swiglu
        self._code = _GATE_CODE[activation_func]

    def forward(self, x, bias=None):
        return _GatedActivationFunction.apply(x, bias, self._code)
