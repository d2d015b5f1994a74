"""LayerNorm and RMSNorm on MI355X.

Surface of GPT-NeoX's ``megatron/model/norms.py``: ``get_norm`` (:19-51),
``LayerNorm`` (:16, torch's class there), ``RMSNorm`` (:54-107, partial variant
included) and ``ScaleNorm`` (:110-119), with the same constructor arguments and
parameter names (``weight`` / ``bias``, ``scale`` / ``offset``, ``g``). Forward and backward are hand-written gfx950 kernels
(libneox_hotpath.so): one pass over the row for the forward, one for the
backward including the parameter gradients. Statistics and arithmetic are fp32
and the result is rounded once, which is what torch's LayerNorm kernel and the
fused RMSNorm variants do; the Python ``RMSNorm`` of the reference, run eagerly
on 16-bit tensors, rounds after every operator and so differs by a few units in
the last place.

The reference's three classes are plain torch modules that work on any device.
That is kept: a tensor that is not on a GPU is normalised with the reference's
own torch expressions (``torch.nn.functional.layer_norm``, the statements of
``RMSNorm.forward`` and ``ScaleNorm.forward``), with autograd's backward. A
tensor on a GPU always takes the kernels; if the library is missing that raises,
there is no torch path for GPU tensors.

Not provided: the Transformer Engine classes (``te_rmsnorm``, ``te_layernorm``).
"""
import numbers

import torch

from ..fused_kernels import _hotpath as _hp


def _ptr(t):
    return None if t is None else t.data_ptr()


def _param_code(x, *params):
    dtypes = {p.dtype for p in params if p is not None}
    if not dtypes:
        return _hp.dtype_code(x, "norm")
    if len(dtypes) > 1:
        raise RuntimeError("norm: the parameters must share one dtype")
    dt = dtypes.pop()
    if dt not in (x.dtype, torch.float32):
        raise RuntimeError(f"norm: parameters must be float32 or {x.dtype}, got {dt}")
    return _hp._DTYPE[dt]


def _check_param(p, cols, x, what):
    if p is None:
        return None
    if p.numel() != cols:
        raise RuntimeError(f"{what}: parameter of {p.numel()} elements for rows of {cols}")
    _hp.require_gpu(p, what)
    return p.contiguous()


def _workspace(rows, cols, code, device):
    nbytes = _hp.lib().nhp_norm_bwd_workspace_bytes(rows, cols, code)
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


class _LayerNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, eps):
        what = "LayerNorm"
        _hp.require_gpu(x, what)
        cols = x.size(-1)
        src = x.contiguous()
        weight = _check_param(weight, cols, x, what)
        bias = _check_param(bias, cols, x, what)
        rows = src.numel() // max(cols, 1)
        y = torch.empty_like(src)
        mean = torch.empty(rows, dtype=torch.float32, device=src.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=src.device)
        code, pcode = _hp.dtype_code(src, what), _param_code(src, weight, bias)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), src.data_ptr(),
                                             _ptr(weight), _ptr(bias), float(eps), rows, cols, code, pcode,
                                             _hp.stream_of(src))
        _hp.check(rc, what)
        ctx.save_for_backward(src, weight, mean, rstd)
        ctx.has_bias = bias is not None
        ctx.codes = (code, pcode)
        return y

    @staticmethod
    def backward(ctx, grad):
        what = "LayerNorm backward"
        src, weight, mean, rstd = ctx.saved_tensors
        g = grad.contiguous()
        cols = src.size(-1)
        rows = src.numel() // max(cols, 1)
        code, pcode = ctx.codes
        want_w = weight is not None and ctx.needs_input_grad[1]
        want_b = ctx.has_bias and ctx.needs_input_grad[2]
        pdtype = weight.dtype if weight is not None else (torch.float32 if pcode == _hp.F32 else src.dtype)
        dx = torch.empty_like(src)
        dw = torch.empty(cols, dtype=pdtype, device=src.device) if want_w else None
        db = torch.empty(cols, dtype=pdtype, device=src.device) if want_b else None
        ws = _workspace(rows, cols, code, src.device) if (want_w or want_b) else None
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_layernorm_bwd(dx.data_ptr(), _ptr(dw), _ptr(db), g.data_ptr(), src.data_ptr(),
                                             mean.data_ptr(), rstd.data_ptr(), _ptr(weight), _ptr(ws), rows, cols,
                                             code, pcode, _hp.stream_of(src))
        _hp.check(rc, what)
        if rows == 0:
            dw = None if dw is None else dw.zero_()
            db = None if db is None else db.zero_()
        return dx, dw, db, None


class _LayerNormPairFunction(torch.autograd.Function):
    """Two LayerNorms of one input: one pass forward (shared statistics, two results) and one pass backward
    (one gradient for the input, the parameter gradients of both)."""

    @staticmethod
    def forward(ctx, x, weight1, bias1, weight2, bias2, eps):
        what = "LayerNorm pair"
        _hp.require_gpu(x, what)
        cols = x.size(-1)
        src = x.contiguous()
        weight1, bias1 = _check_param(weight1, cols, x, what), _check_param(bias1, cols, x, what)
        weight2, bias2 = _check_param(weight2, cols, x, what), _check_param(bias2, cols, x, what)
        rows = src.numel() // max(cols, 1)
        y1, y2 = torch.empty_like(src), torch.empty_like(src)
        mean = torch.empty(rows, dtype=torch.float32, device=src.device)
        rstd = torch.empty(rows, dtype=torch.float32, device=src.device)
        code, pcode = _hp.dtype_code(src, what), _param_code(src, weight1, bias1, weight2, bias2)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_layernorm_pair_fwd(y1.data_ptr(), y2.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                                                  src.data_ptr(), _ptr(weight1), _ptr(bias1), _ptr(weight2), _ptr(bias2),
                                                  float(eps), rows, cols, code, pcode, _hp.stream_of(src))
        _hp.check(rc, what)
        ctx.save_for_backward(src, weight1, weight2, mean, rstd)
        ctx.has_bias = (bias1 is not None, bias2 is not None)
        ctx.codes = (code, pcode)
        return y1, y2

    @staticmethod
    def backward(ctx, grad1, grad2):
        what = "LayerNorm pair backward"
        src, weight1, weight2, mean, rstd = ctx.saved_tensors
        cols = src.size(-1)
        rows = src.numel() // max(cols, 1)
        code, pcode = ctx.codes
        g1 = torch.zeros_like(src) if grad1 is None else grad1.contiguous()
        g2 = torch.zeros_like(src) if grad2 is None else grad2.contiguous()
        needs = ctx.needs_input_grad
        pdtype = torch.float32 if pcode == _hp.F32 else src.dtype

        def new(wanted):
            return torch.empty(cols, dtype=pdtype, device=src.device) if wanted else None

        dw1, db1 = new(weight1 is not None and needs[1]), new(ctx.has_bias[0] and needs[2])
        dw2, db2 = new(weight2 is not None and needs[3]), new(ctx.has_bias[1] and needs[4])
        dx = torch.empty_like(src)
        ws = None
        if any(t is not None for t in (dw1, db1, dw2, db2)):
            nbytes = _hp.lib().nhp_layernorm_pair_bwd_workspace_bytes(rows, cols, code)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=src.device) if nbytes else None
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_layernorm_pair_bwd(dx.data_ptr(), _ptr(dw1), _ptr(db1), _ptr(dw2), _ptr(db2), g1.data_ptr(),
                                                  g2.data_ptr(), src.data_ptr(), mean.data_ptr(), rstd.data_ptr(),
                                                  _ptr(weight1), _ptr(weight2), _ptr(ws), rows, cols, code, pcode,
                                                  _hp.stream_of(src))
        _hp.check(rc, what)
        if rows == 0:
            for t in (dw1, db1, dw2, db2):
                if t is not None:
                    t.zero_()
        return dx, dw1, db1, dw2, db2, None


def layer_norm_pair(x, norm_a, norm_b):
    """``(norm_a(x), norm_b(x))`` for two ``LayerNorm`` modules of this file applied to the same input, in one
    kernel each way when their settings allow it (same epsilon, rows of at most 16 KiB), otherwise as two
    separate calls. The parallel-residual transformer layer does this with its input and post-attention
    norms (megatron/model/transformer.py:1195-1213)."""
    same = (isinstance(norm_a, LayerNorm) and isinstance(norm_b, LayerNorm) and norm_a.eps == norm_b.eps
            and norm_a.normalized_shape == norm_b.normalized_shape and x.size(-1) == norm_a.normalized_shape[0]
            and x.size(-1) * x.element_size() <= 16384)
    if not same:
        return norm_a(x), norm_b(x)
    return _LayerNormPairFunction.apply(x, norm_a.weight, norm_a.bias, norm_b.weight, norm_b.bias, norm_a.eps)


class LayerNorm(torch.nn.Module):
    """``torch.nn.LayerNorm`` over the last dimension (what ``get_norm`` returns for ``norm: layernorm``)."""

    def __init__(self, normalized_shape, eps=1e-5, elementwise_affine=True, bias=True, device=None, dtype=None):
        super().__init__()
        if isinstance(normalized_shape, numbers.Integral):
            normalized_shape = (int(normalized_shape),)
        if len(normalized_shape) != 1:
            raise NotImplementedError("only normalisation over the last dimension is provided")
        self.normalized_shape = tuple(normalized_shape)
        self.eps = eps
        self.elementwise_affine = elementwise_affine
        if elementwise_affine:
            self.weight = torch.nn.Parameter(torch.ones(self.normalized_shape, device=device, dtype=dtype))
            if bias:
                self.bias = torch.nn.Parameter(torch.zeros(self.normalized_shape, device=device, dtype=dtype))
            else:
                self.register_parameter("bias", None)
        else:
            self.register_parameter("weight", None)
            self.register_parameter("bias", None)

    def forward(self, input):
        if input.size(-1) != self.normalized_shape[0]:
            raise RuntimeError(f"LayerNorm: expected last dimension {self.normalized_shape[0]}, got {input.size(-1)}")
        if input.device.type != "cuda":
            # off the GPU: torch's own LayerNorm, which is the reference's class (megatron/model/norms.py:16)
            return torch.nn.functional.layer_norm(input, self.normalized_shape, self.weight, self.bias, self.eps)
        return _LayerNormFunction.apply(input, self.weight, self.bias, self.eps)

    def extra_repr(self):
        return f"{self.normalized_shape}, eps={self.eps}, elementwise_affine={self.elementwise_affine}"


class _RMSNormFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, scale, offset, eps, eps_mode, stat_cols=None):
        what = "RMSNorm"
        _hp.require_gpu(x, what)
        cols = x.size(-1)
        src = x.contiguous()
        scale = _check_param(scale, cols, x, what)
        offset = _check_param(offset, cols, x, what)
        rows = src.numel() // max(cols, 1)
        y = torch.empty_like(src)
        inv = torch.empty(rows, dtype=torch.float32, device=src.device)
        code, pcode = _hp.dtype_code(src, what), _param_code(src, scale, offset)
        stat = cols if stat_cols is None else int(stat_cols)
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_rmsnorm_partial_fwd(y.data_ptr(), inv.data_ptr(), src.data_ptr(), _ptr(scale),
                                                   _ptr(offset), float(eps), int(eps_mode), rows, cols, stat, code,
                                                   pcode, _hp.stream_of(src))
        _hp.check(rc, what)
        ctx.save_for_backward(src, scale, inv)
        ctx.has_offset = offset is not None
        ctx.conf = (code, pcode, float(eps), int(eps_mode), stat)
        return y

    @staticmethod
    def backward(ctx, grad):
        what = "RMSNorm backward"
        src, scale, inv = ctx.saved_tensors
        g = grad.contiguous()
        cols = src.size(-1)
        rows = src.numel() // max(cols, 1)
        code, pcode, eps, eps_mode, stat = ctx.conf
        want_s = scale is not None and ctx.needs_input_grad[1]
        want_o = ctx.has_offset and ctx.needs_input_grad[2]
        pdtype = scale.dtype if scale is not None else (torch.float32 if pcode == _hp.F32 else src.dtype)
        dx = torch.empty_like(src)
        ds = torch.empty(cols, dtype=pdtype, device=src.device) if want_s else None
        do = torch.empty(cols, dtype=pdtype, device=src.device) if want_o else None
        ws = _workspace(rows, cols, code, src.device) if (want_s or want_o) else None
        with _hp.device_guard(src):
            rc = _hp.lib().nhp_rmsnorm_partial_bwd(dx.data_ptr(), _ptr(ds), _ptr(do), g.data_ptr(), src.data_ptr(),
                                                   inv.data_ptr(), _ptr(scale), _ptr(ws), eps, eps_mode, rows, cols,
                                                   stat, code, pcode, _hp.stream_of(src))
        _hp.check(rc, what)
        if rows == 0:
            ds = None if ds is None else ds.zero_()
            do = None if do is None else do.zero_()
        return dx, ds, do, None, None, None


class RMSNorm(torch.nn.Module):
    """Root-mean-square normalisation, ``scale * x / (rms(x) + eps) [+ offset]``
    (the reference's Python class, megatron/model/norms.py:54-107). With
    ``0 <= p <= 1`` the rms is taken over the first ``int(dim * p)`` features only
    (partial RMSNorm, :87-94).

    ``fused_eps=True`` selects the other definition the reference knows,
    ``scale * x * rsqrt(mean(x^2) + eps)`` (MixedFusedRMSNorm)."""

    def __init__(self, dim, p=-1.0, eps=1e-8, bias=False, fused_eps=False):
        super().__init__()
        self.partial_size = None
        if 0.0 <= p <= 1.0:
            self.partial_size = int(dim * p)
            if self.partial_size < 1:
                # the reference divides by zero here (0 ** -0.5)
                raise ZeroDivisionError(f"partial RMSNorm: int({dim} * {p}) = 0 features to take the rms of")
        self.eps = eps
        self.d = dim
        self.p = p
        self.bias = bias
        self.fused_eps = fused_eps
        self.scale = torch.nn.Parameter(torch.ones(dim))
        if self.bias:
            self.offset = torch.nn.Parameter(torch.zeros(dim))
        else:
            self.register_parameter("offset", None)

    def forward(self, x):
        if x.size(-1) != self.d:
            raise RuntimeError(f"RMSNorm: expected last dimension {self.d}, got {x.size(-1)}")
        if x.device.type != "cuda":
            return self._forward_torch(x)
        return _RMSNormFunction.apply(x, self.scale, self.offset, self.eps, 0 if self.fused_eps else 1,
                                      self.partial_size)

    def _forward_torch(self, x):
        """Off the GPU: the statements of the reference's ``RMSNorm.forward`` (megatron/model/norms.py:82-107), every
        operator in the tensors' own dtypes; with ``fused_eps`` the fused definition evaluated in fp32."""
        if self.fused_eps:
            stat = x.float() if self.partial_size is None else x.float()[..., : self.partial_size]
            inv = torch.rsqrt(stat.pow(2).mean(dim=-1, keepdim=True) + self.eps)
            out = x.float() * inv * self.scale.float()
            if self.offset is not None:
                out = out + self.offset.float()
            return out.to(x.dtype)
        measured = x if self.partial_size is None else x[..., : self.partial_size]
        count = self.d if self.partial_size is None else self.partial_size
        rms = measured.norm(2, dim=-1, keepdim=True) * count ** -0.5
        normed = x / (rms + self.eps)
        if self.offset is not None:
            return self.scale * normed + self.offset  # the reference does not cast back on this branch
        return (self.scale * normed).to(x.dtype)


class ScaleNorm(torch.nn.Module):
    """``x / clamp(||x||_2, min=eps) * g`` with one learned scalar ``g``
    (megatron/model/norms.py:110-119). Runs on the RMSNorm kernels: the scalar is
    handed over as a vector of equal values, and its gradient is the sum of that
    vector's gradient (autograd does both through ``expand``)."""

    def __init__(self, dim, eps=1e-5):
        super().__init__()
        self.g = torch.nn.Parameter(torch.ones(1))
        self.eps = eps

    def forward(self, x):
        if x.device.type != "cuda":
            # off the GPU: the reference's two statements (megatron/model/norms.py:116-119)
            return x / torch.norm(x, dim=-1, keepdim=True).clamp(min=self.eps) * self.g
        g = self.g if self.g.dtype in (x.dtype, torch.float32) else self.g.to(x.dtype)
        return _RMSNormFunction.apply(x, g.expand(x.size(-1)), None, self.eps, 2, None)


def get_norm(neox_args):
    """(norm class, eps) for ``neox_args.norm`` in {"layernorm", "rmsnorm", "scalenorm"}
    (megatron/model/norms.py:19-51); the ``*_fusion`` flags select the classes of
    ``fused_layer_norm``, which run on the same kernels."""
    if neox_args.norm == "rmsnorm":
        if getattr(neox_args, "rmsnorm_fusion", False):
            from .fused_layer_norm import MixedFusedRMSNorm

            return MixedFusedRMSNorm, neox_args.rms_norm_epsilon
        return RMSNorm, neox_args.rms_norm_epsilon
    if neox_args.norm == "layernorm":
        if getattr(neox_args, "layernorm_fusion", False):
            from .fused_layer_norm import MixedFusedLayerNorm

            return MixedFusedLayerNorm, neox_args.layernorm_epsilon
        return LayerNorm, neox_args.layernorm_epsilon
    if neox_args.norm == "scalenorm":
        return ScaleNorm, neox_args.scalenorm_epsilon
    raise ValueError(f"norm {neox_args.norm} not provided by the MI355X kernels")
