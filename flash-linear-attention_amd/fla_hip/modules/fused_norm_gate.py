"""Layer / RMS normalisation with a swish or sigmoid output gate, with the reference's interface:
``layer_norm_gated_fwd`` / ``layer_norm_gated_bwd`` (fla/modules/fused_norm_gate.py:456-538, :541-650), the autograd
function over them (:653-746), ``layer_norm_gated`` / ``rms_norm_gated`` (:836-883) and the ``FusedRMSNormGated`` /
``FusedLayerNormGated`` layers (:940-1105).  All compute is done by ``gdn_norm_gated_fwd`` and ``gdn_norm_gated_bwd`` of
the HIP library."""
from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import current_stream_ptr, dtype_code, forward_only, ptr, require_gpu


def _gate_code(activation: str) -> int:
    if activation in ('swish', 'silu'):
        return _lib.ACT_SILU
    if activation == 'sigmoid':
        return _lib.ACT_SIGMOID
    raise ValueError(f'Unsupported activation: {activation}')


def layer_norm_gated_fwd(
    x: torch.Tensor,
    g: torch.Tensor,
    weight: torch.Tensor | None,
    bias: torch.Tensor | None,
    activation: str = 'swish',
    eps: float = 1e-5,
    residual: torch.Tensor | None = None,
    out_dtype: torch.dtype | None = None,
    residual_dtype: torch.dtype | None = None,
    is_rms_norm: bool = False,
):
    """``x``, ``g`` are ``[T, D]``.  Returns ``(y, mean, rstd, residual_out)`` like the reference: ``mean`` is ``None``
    for RMS norm and ``residual_out`` is ``x`` itself when no residual stream was asked for."""
    dev = require_gpu(x, g)
    forward_only('layer_norm_gated', x, g, residual)
    if x.dim() != 2 or g.shape != x.shape:
        raise ValueError(f'x and g must be [T, D] and alike, got {tuple(x.shape)} and {tuple(g.shape)}')
    T, D = x.shape
    if residual is not None:
        residual_dtype = residual.dtype
        assert residual.shape == (T, D)
        residual = residual.contiguous()
    if weight is not None:
        assert weight.shape == (D,)
    if bias is not None:
        assert bias.shape == (D,)
    if D * x.element_size() >= 65536:
        raise RuntimeError("This layer norm doesn't support feature dim >= 64KB.")
    x = x.contiguous()
    g = g.to(x.dtype).contiguous()
    y = torch.empty_like(x)
    if residual is not None or (residual_dtype is not None and residual_dtype != x.dtype):
        residual_out = torch.empty(T, D, device=dev, dtype=residual_dtype)
    else:
        residual_out = None
    mean = torch.empty((T,), dtype=torch.float, device=dev) if not is_rms_norm else None
    rstd = torch.empty((T,), dtype=torch.float, device=dev)
    if weight is not None and bias is not None and bias.dtype != weight.dtype:
        bias = bias.to(weight.dtype)
    params = weight if weight is not None else bias
    with torch.cuda.device(dev):
        _lib.check(_lib.load().gdn_norm_gated_fwd(
            ptr(x), ptr(g), ptr(weight), ptr(bias), ptr(residual), ptr(y), ptr(residual_out), ptr(mean), ptr(rstd),
            T, D, float(eps),
            dtype_code(x.dtype), dtype_code(params.dtype) if params is not None else _lib.DTYPE_F32,
            dtype_code(residual.dtype) if residual is not None else _lib.DTYPE_F32,
            dtype_code(residual_out.dtype) if residual_out is not None else _lib.DTYPE_F32,
            _gate_code(activation), int(bool(is_rms_norm)), current_stream_ptr(dev)))
    if out_dtype is not None and out_dtype != y.dtype:
        y = y.to(out_dtype)
    return y, mean, rstd, residual_out if residual_out is not None else x


def layer_norm_gated_bwd(
    dy: torch.Tensor,
    x: torch.Tensor,
    g: torch.Tensor,
    weight: torch.Tensor | None,
    bias: torch.Tensor | None,
    activation: str = 'swish',
    eps: float = 1e-5,
    mean: torch.Tensor | None = None,
    rstd: torch.Tensor | None = None,
    dresidual: torch.Tensor | None = None,
    has_residual: bool = False,
    is_rms_norm: bool = False,
    x_dtype: torch.dtype | None = None,
    recompute_output: bool = False,
):
    """Gradients ``(dx, dg, dw, db, dresidual_in)`` of ``layer_norm_gated_fwd``.  ``x`` is what was normalised (the forward's
    fourth result), ``mean`` / ``rstd`` the forward's row statistics, ``dresidual`` the gradient of the residual stream
    handed on (prenorm).  ``dx`` and ``dg`` come in ``x_dtype`` (default: x's own); ``dresidual_in`` is ``None`` unless
    ``has_residual``.  The kernel computes in x's dtype: g, dy and dresidual of another dtype are converted first."""
    if recompute_output:
        raise NotImplementedError('recompute_output belongs to the fused norm + linear layer, which is not part of this build')
    dev = require_gpu(dy, x, g)
    T, D = x.shape
    if dy.shape != (T, D) or g.shape != (T, D):
        raise ValueError(f'dy, x and g must be [T, D] and alike, got {tuple(dy.shape)}, {tuple(x.shape)}, {tuple(g.shape)}')
    vec = 16 // x.element_size()
    ld = (D + vec - 1) // vec * vec
    if ld > 2048:
        raise NotImplementedError(f'the backward of the gated norm covers feature dims up to 2048 (got {D})')
    if rstd is None or (mean is None and not is_rms_norm):
        raise ValueError('layer_norm_gated_bwd needs the row statistics of the forward (rstd, and mean for layer norm)')

    def rows(t):                                                # [T, ld] in x's dtype, zeros from D on
        t = t.reshape(T, D).to(x.dtype)
        return F.pad(t, (0, ld - D)) if ld != D else t.contiguous()

    x_k, g_k, dy_k = rows(x), rows(g), rows(dy)
    dres_k = None if dresidual is None else rows(dresidual)
    if weight is not None and bias is not None and bias.dtype != weight.dtype:
        bias = bias.to(weight.dtype)
    params = weight if weight is not None else bias
    dx = torch.empty_like(x_k)
    dg = torch.empty_like(x_k)
    parts = max(1, min(1024, (T + 31) // 32))
    dw_part = torch.empty(parts, ld, dtype=torch.float32, device=dev) if weight is not None else None
    db_part = torch.empty(parts, ld, dtype=torch.float32, device=dev) if bias is not None else None
    with torch.cuda.device(dev):
        _lib.check(_lib.load().gdn_norm_gated_bwd(
            ptr(dy_k), ptr(x_k), ptr(g_k), ptr(weight), ptr(bias), ptr(mean), ptr(rstd), ptr(dres_k), ptr(dx), ptr(dg),
            ptr(dw_part), ptr(db_part), T, D, ld, parts, dtype_code(x.dtype),
            dtype_code(params.dtype) if params is not None else _lib.DTYPE_F32,
            _gate_code(activation), int(bool(is_rms_norm)), current_stream_ptr(dev)))
    dw = dw_part.sum(0)[:D].to(weight.dtype) if weight is not None else None
    db = db_part.sum(0)[:D].to(bias.dtype) if bias is not None else None
    if ld != D:
        dx, dg = dx[:, :D].contiguous(), dg[:, :D].contiguous()
    dresidual_in = dx if has_residual else None
    if x_dtype is not None and x_dtype != dx.dtype:
        dx, dg = dx.to(x_dtype), dg.to(x_dtype)
    return dx, dg, dw, db, dresidual_in


class LayerNormGatedFunction(torch.autograd.Function):
    """Forward and backward kernels as one differentiable function (fla/modules/fused_norm_gate.py:653-746)."""

    @staticmethod
    def forward(ctx, x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, is_rms_norm):
        x_shape_og, g_shape_og = x.shape, g.shape
        x2 = x.reshape(-1, x.shape[-1])
        g2 = g.reshape(-1, g.shape[-1])
        if residual is not None:
            assert residual.shape == x_shape_og
            residual = residual.reshape(-1, residual.shape[-1])
        residual_dtype = residual.dtype if residual is not None else (torch.float if residual_in_fp32 else None)
        y, mean, rstd, residual_out = layer_norm_gated_fwd(
            x=x2, g=g2, weight=weight, bias=bias, activation=activation, eps=eps, residual=residual,
            residual_dtype=residual_dtype, is_rms_norm=is_rms_norm)
        ctx.save_for_backward(residual_out, g2, weight, bias, mean, rstd)
        ctx.x_shape_og, ctx.g_shape_og = x_shape_og, g_shape_og
        ctx.activation, ctx.eps, ctx.is_rms_norm = activation, eps, is_rms_norm
        ctx.has_residual = residual is not None
        ctx.residual_dtype = residual.dtype if residual is not None else None
        ctx.prenorm = prenorm
        ctx.x_dtype, ctx.g_dtype = x.dtype, g.dtype
        y = y.reshape(x_shape_og)
        return y if not prenorm else (y, residual_out.reshape(x_shape_og))

    @staticmethod
    def backward(ctx, dy, *args):
        x, g, weight, bias, mean, rstd = ctx.saved_tensors
        dy = dy.reshape(-1, dy.shape[-1])
        dresidual = args[0].reshape(-1, args[0].shape[-1]) if ctx.prenorm and args and args[0] is not None else None
        dx, dg, dw, db, dres_in = layer_norm_gated_bwd(
            dy=dy, x=x, g=g, weight=weight, bias=bias, activation=ctx.activation, eps=ctx.eps, mean=mean, rstd=rstd,
            dresidual=dresidual, has_residual=ctx.has_residual, is_rms_norm=ctx.is_rms_norm, x_dtype=ctx.x_dtype)
        if dg.dtype != ctx.g_dtype:
            dg = dg.to(ctx.g_dtype)
        if dres_in is not None:
            dres_in = dres_in.to(ctx.residual_dtype).reshape(ctx.x_shape_og)
        return dx.reshape(ctx.x_shape_og), dg.reshape(ctx.g_shape_og), dw, db, None, dres_in, None, None, None, None


def _norm_gated(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, is_rms_norm):
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, g, weight, bias, residual)):
        return LayerNormGatedFunction.apply(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, is_rms_norm)
    x_shape_og = x.shape
    x = x.reshape(-1, x.shape[-1])
    g = g.reshape(-1, g.shape[-1])
    if residual is not None:
        assert residual.shape == x_shape_og
        residual = residual.reshape(-1, residual.shape[-1])
    residual_dtype = residual.dtype if residual is not None else (torch.float if residual_in_fp32 else None)
    y, _, _, residual_out = layer_norm_gated_fwd(
        x=x, g=g, weight=weight, bias=bias, activation=activation, eps=eps, residual=residual,
        residual_dtype=residual_dtype, is_rms_norm=is_rms_norm)
    y = y.reshape(x_shape_og)
    return y if not prenorm else (y, residual_out.reshape(x_shape_og))


def layer_norm_gated(
    x: torch.Tensor,
    g: torch.Tensor,
    weight: torch.Tensor | None,
    bias: torch.Tensor | None,
    activation: str = 'swish',
    residual: torch.Tensor | None = None,
    prenorm: bool = False,
    residual_in_fp32: bool = False,
    eps: float = 1e-6,
):
    return _norm_gated(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, False)


def rms_norm_gated(
    x: torch.Tensor,
    g: torch.Tensor,
    weight: torch.Tensor | None,
    bias: torch.Tensor | None,
    activation: str = 'swish',
    residual: torch.Tensor | None = None,
    prenorm: bool = False,
    residual_in_fp32: bool = False,
    eps: float = 1e-6,
):
    return _norm_gated(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, True)


class _NormGated(nn.Module):
    _is_rms = False

    def _setup(self, hidden_size, elementwise_affine, bias, activation, eps, device, dtype):
        factory_kwargs = {'device': device, 'dtype': dtype}
        self.hidden_size = hidden_size
        self.elementwise_affine = elementwise_affine
        self.eps = eps
        self.activation = activation
        if self.activation not in ['swish', 'silu', 'sigmoid']:
            raise ValueError(f'Unsupported activation: {self.activation}')
        self.register_parameter('weight', None)
        self.register_parameter('bias', None)
        if elementwise_affine:
            self.weight = nn.Parameter(torch.empty(hidden_size, **factory_kwargs))
            if bias:
                self.bias = nn.Parameter(torch.empty(hidden_size, **factory_kwargs))
        self.reset_parameters()

    def reset_parameters(self):
        if self.elementwise_affine:
            nn.init.ones_(self.weight)
            if self.bias is not None:
                nn.init.zeros_(self.bias)

    def __repr__(self) -> str:
        s = f'{self.__class__.__name__}({self.hidden_size}'
        if not self.elementwise_affine:
            s += f', elementwise_affine={self.elementwise_affine}'
        return s + f', eps={self.eps}, activation={self.activation})'

    def forward(
        self,
        x: torch.Tensor,
        g: torch.Tensor,
        residual: torch.Tensor | None = None,
        prenorm: bool = False,
        residual_in_fp32: bool = False,
    ) -> torch.Tensor:
        return _norm_gated(x, g, self.weight, self.bias, self.activation, residual, self.eps, prenorm,
                           residual_in_fp32, self._is_rms)


class FusedLayerNormGated(_NormGated):
    """fla/modules/fused_norm_gate.py:940-1004"""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, bias: bool = False,
                 activation: str = 'swish', eps: float = 1e-5, device=None, dtype=None):
        super().__init__()
        self._setup(hidden_size, elementwise_affine, bias, activation, eps, device, dtype)


class FusedRMSNormGated(_NormGated):
    """fla/modules/fused_norm_gate.py:1007-1067 (never a bias)"""
    _is_rms = True

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5,
                 activation: str = 'swish', device=None, dtype=None):
        super().__init__()
        self._setup(hidden_size, elementwise_affine, False, activation, eps, device, dtype)


class FusedLayerNormSwishGate(FusedLayerNormGated):
    """fla/modules/fused_norm_gate.py:1070-1087"""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, bias: bool = False, eps: float = 1e-5,
                 device=None, dtype=None):
        super().__init__(hidden_size=hidden_size, elementwise_affine=elementwise_affine, bias=bias, eps=eps,
                         device=device, dtype=dtype)


class FusedRMSNormSwishGate(FusedRMSNormGated):
    """fla/modules/fused_norm_gate.py:1090-1105"""

    def __init__(self, hidden_size: int, elementwise_affine: bool = True, eps: float = 1e-5, device=None, dtype=None):
        super().__init__(hidden_size=hidden_size, elementwise_affine=elementwise_affine, eps=eps,
                         device=device, dtype=dtype)
