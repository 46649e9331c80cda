"""Layer / RMS normalisation with a swish or sigmoid output gate, forward only, with the reference's interface:
``layer_norm_gated_fwd`` (fla/modules/fused_norm_gate.py:456-538), ``layer_norm_gated`` / ``rms_norm_gated``
(:836-883) and the ``FusedRMSNormGated`` / ``FusedLayerNormGated`` layers (:940-1105).  All compute is done by
``gdn_norm_gated_fwd`` of the HIP library."""
from __future__ import annotations

import torch
import torch.nn as nn

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


def _norm_gated(x, g, weight, bias, activation, residual, eps, prenorm, residual_in_fp32, is_rms_norm):
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
