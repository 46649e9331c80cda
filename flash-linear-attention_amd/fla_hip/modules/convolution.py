"""Causal depthwise short convolution with the reference's interface:
``causal_conv1d`` (fla/modules/conv/causal_conv1d.py:16-129), ``causal_conv1d_fwd``, ``causal_conv1d_bwd``,
``causal_conv1d_update_states``, ``causal_conv1d_update`` (fla/modules/conv/triton/ops.py:37-96, :147-249,
:252-296, :301-363), the autograd function that ties forward and backward together (:366-428) and the
``ShortConvolution`` layer (fla/modules/conv/short_conv.py:24-250).  All compute is done by ``gdn_causal_conv1d_fwd``,
``gdn_causal_conv1d_bwd`` and ``gdn_causal_conv1d_update`` of the HIP library; the one-token update is forward only."""
from __future__ import annotations

import os
import warnings

import torch
import torch.nn as nn
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import current_stream_ptr, dtype_code, forward_only, ptr, require_gpu
from fla_hip.ops.utils.index import check_cu_seqlens, prepare_chunk_indices
from fla_hip.utils import input_guard

MAX_KERNEL_SIZE = 8


def _activation_code(activation: str | None) -> int:
    if activation is None:
        return _lib.ACT_NONE
    if activation in ('swish', 'silu'):
        return _lib.ACT_SILU
    raise NotImplementedError(f'activation `{activation}` is not supported (None, `swish`, `silu`)')


def _rows(x: torch.Tensor, D: int) -> torch.Tensor:
    """[B, T, ...] -> [B, T, D] with adjacent channels; other strides are kept (a slice of a wider projection is
    read in place, as the reference's kernel does through its stride arguments)."""
    if x.dim() != 3 or x.shape[-1] != D:
        x = x.reshape(x.shape[0], x.shape[1], -1)
    if x.shape[-1] != D:
        raise ValueError(f'x has {x.shape[-1]} channels, the weight has {D}')
    if x.stride(-1) != 1 or (x.shape[1] > 1 and x.stride(1) < D):
        x = x.contiguous()
    return x


def _launch_fwd(x, weight, bias, residual, initial_state, want_y, want_state, activation, cu_seqlens, W):
    dev = require_gpu(x)
    forward_only('causal_conv1d', x, residual)
    B, T, D = x.shape
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    if cu_seqlens is not None and B != 1:
        raise ValueError(f'The batch size is expected to be 1 rather than {B} when using `cu_seqlens`.')
    if initial_state is not None:
        if tuple(initial_state.shape) != (N, D, W):
            raise ValueError(f'initial_state must be [{N}, {D}, {W}], got {tuple(initial_state.shape)}')
        initial_state = initial_state.contiguous()
    if bias is not None and bias.numel() != D:
        raise ValueError(f'bias must have {D} entries, got {bias.numel()}')
    flags = 0
    if cu_seqlens is not None:
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        elif cu_seqlens.dtype != torch.int64:
            raise ValueError(f'cu_seqlens must be int32 or int64, got {cu_seqlens.dtype}')
        cu_seqlens = cu_seqlens.to(dev).contiguous()
    y = torch.empty(B, T, D, dtype=x.dtype, device=dev) if want_y else None
    final_state = torch.empty(N, D, W, dtype=x.dtype, device=dev) if want_state else None
    if residual is not None:
        residual = residual.reshape(B, T, D).to(x.dtype).contiguous()
    w_dtype = dtype_code(weight.dtype) if weight is not None else _lib.DTYPE_F32
    if bias is not None and weight is not None and bias.dtype != weight.dtype:
        bias = bias.to(weight.dtype)
    with torch.cuda.device(dev):
        _lib.check(_lib.load().gdn_causal_conv1d_fwd(
            ptr(x), ptr(weight), ptr(bias), ptr(residual), ptr(initial_state), ptr(y), ptr(final_state), ptr(cu_seqlens),
            B, T, D, W, N, x.stride(0) if B > 1 else T * max(x.stride(1), D), x.stride(1) if T > 1 else D,
            dtype_code(x.dtype), w_dtype,
            dtype_code(initial_state.dtype) if initial_state is not None else _lib.DTYPE_F32,
            _activation_code(activation), flags, current_stream_ptr(dev)))
    return y, final_state


@input_guard(no_guard_contiguous=['x'])
def causal_conv1d_fwd(
    x: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor | None,
    residual: torch.Tensor | None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    activation: str | None = None,
    cu_seqlens: torch.LongTensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
    chunk_indices: torch.LongTensor | None = None,
    BT: int = 64,
    layout_fallback: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``y`` like ``x`` and, on request, the state ``[N, D, W]`` holding the last ``W`` inputs of every sequence.
    ``cu_seqlens_cpu``, ``chunk_indices``, ``BT`` and ``layout_fallback`` steer the reference's tiling only and
    are accepted for compatibility: the kernel finds sequence boundaries from ``cu_seqlens`` itself."""
    if weight is None:
        raise ValueError('causal_conv1d_fwd needs a weight of shape [D, W]')
    shape = x.shape
    D, W = weight.shape
    if W > MAX_KERNEL_SIZE:
        raise NotImplementedError(f'kernel sizes above {MAX_KERNEL_SIZE} are not supported (got {W})')
    x = _rows(x, D)
    y, final_state = _launch_fwd(x, weight, bias, residual, initial_state, True, bool(output_final_state),
                                 activation, cu_seqlens, W)
    return y.view(shape), final_state


def causal_conv1d_bwd(
    x: torch.Tensor,
    dy: torch.Tensor,
    dht: torch.Tensor | None,
    weight: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    residual: torch.Tensor | None = None,
    initial_state: torch.Tensor | None = None,
    activation: str | None = None,
    cu_seqlens: torch.Tensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
    chunk_indices: torch.LongTensor | None = None,
    BT: int = 64,
    layout_fallback: bool = False,
):
    """Gradients ``(dx, dw, db, dr, dh0)`` of ``causal_conv1d_fwd`` for the output gradient ``dy`` and the gradient ``dht``
    of the final state (``None``: none); ``dr`` is ``dy`` itself when there was a residual, ``dh0`` has the initial
    state's dtype.  ``chunk_indices``, ``BT`` and ``layout_fallback`` steer the reference's tiling only and are accepted for
    compatibility, as in the forward."""
    if weight is None:
        raise ValueError('causal_conv1d_bwd needs the weight of shape [D, W]')
    dev = require_gpu(x, dy)
    shape = x.shape
    D, W = weight.shape
    x = _rows(x, D)
    B, T, _ = x.shape
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    if cu_seqlens is not None and B != 1:
        raise ValueError(f'The batch size is expected to be 1 rather than {B} when using `cu_seqlens`.')
    for name, t, want in (('bias', bias, (D,)), ('initial_state', initial_state, (N, D, W)), ('dht', dht, (N, D, W))):
        if t is not None and tuple(t.shape) != want:
            raise ValueError(f'{name} must have shape {want}, got {tuple(t.shape)}')
    dy = dy.reshape(B, T, D).to(x.dtype).contiguous()
    pad = -D % 4
    if pad or x.data_ptr() % (4 * x.element_size()) or x.stride(1) % 4 or x.stride(0) % 4:
        # the kernel takes four adjacent channels per thread: bring other layouts to that form
        x = F.pad(x, (0, pad)) if pad else x.clone(memory_format=torch.contiguous_format)
        dy = F.pad(dy, (0, pad))
        weight_k = F.pad(weight, (0, 0, 0, pad))
        bias_k = None if bias is None else F.pad(bias, (0, pad))
        h0_k = None if initial_state is None else F.pad(initial_state, (0, 0, 0, pad))
        dht_k = None if dht is None else F.pad(dht, (0, 0, 0, pad))
    else:
        weight_k, bias_k, h0_k, dht_k = weight, bias, initial_state, dht
    Dk = D + pad
    weight_k = weight_k.contiguous()
    if bias_k is not None:
        bias_k = bias_k.to(weight_k.dtype).contiguous()
    if h0_k is not None:
        h0_k = h0_k.contiguous()
    if dht_k is not None:
        dht_k = dht_k.to(x.dtype).contiguous()
    flags = 0
    tile_table = None
    if cu_seqlens is not None:
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        elif cu_seqlens.dtype != torch.int64:
            raise ValueError(f'cu_seqlens must be int32 or int64, got {cu_seqlens.dtype}')
        cu_seqlens = cu_seqlens.to(dev).contiguous()
        # (a caller's chunk_indices may have been made for another tile size: the kernel's 64-token tiles are derived here)
        check_cu_seqlens(cu_seqlens, T, cu_seqlens_cpu)
        tile_table = prepare_chunk_indices(cu_seqlens, 64, cu_seqlens_cpu=cu_seqlens_cpu)
        tile_table = tile_table.to(device=dev, dtype=cu_seqlens.dtype).contiguous()
        num_tiles = tile_table.shape[0]
        dx = torch.zeros(B, T, Dk, dtype=x.dtype, device=dev)   # tokens outside the sequences keep a zero gradient
    else:
        num_tiles = B * ((T + 63) // 64)
        dx = torch.empty(B, T, Dk, dtype=x.dtype, device=dev)
    parts = (num_tiles + _lib.CONV_BWD_TILES_PER_PART - 1) // _lib.CONV_BWD_TILES_PER_PART
    dw_part = torch.empty(max(parts, 1), Dk, W, dtype=torch.float32, device=dev)
    db_part = torch.empty(max(parts, 1), Dk, dtype=torch.float32, device=dev) if bias_k is not None else None
    if parts == 0:
        dw_part.zero_()
        if db_part is not None:
            db_part.zero_()
    dh0 = torch.empty(N, Dk, W, dtype=torch.float32, device=dev) if initial_state is not None else None
    with torch.cuda.device(dev):
        _lib.check(_lib.load().gdn_causal_conv1d_bwd(
            ptr(x), ptr(weight_k), ptr(bias_k), ptr(h0_k), ptr(dy), ptr(dht_k), ptr(dx), ptr(dw_part), ptr(db_part), ptr(dh0),
            ptr(cu_seqlens), ptr(tile_table), B, T, Dk, W, N, num_tiles,
            x.stride(0) if B > 1 else T * max(x.stride(1), Dk), x.stride(1) if T > 1 else Dk,
            dtype_code(x.dtype), dtype_code(weight_k.dtype),
            dtype_code(h0_k.dtype) if h0_k is not None else _lib.DTYPE_F32,
            _activation_code(activation), flags, current_stream_ptr(dev)))
    dw = dw_part.sum(0)[:D].to(weight.dtype)
    db = db_part.sum(0)[:D].to(bias.dtype) if bias is not None else None
    if pad:
        dx = dx[..., :D].contiguous()
    if dh0 is not None:
        dh0 = dh0[:, :D].to(initial_state.dtype)
    dr = dy[..., :D].reshape(shape) if residual is not None else None
    return dx.view(shape), dw, db, dr, dh0


class CausalConv1dFunction(torch.autograd.Function):
    """Forward and backward kernels as one differentiable function (fla/modules/conv/triton/ops.py:366-428)."""

    @staticmethod
    def forward(ctx, x, weight, bias, residual, initial_state, output_final_state, activation, cu_seqlens, cu_seqlens_cpu,
                chunk_indices):
        ctx.activation = activation
        ctx.cu_seqlens = cu_seqlens
        ctx.cu_seqlens_cpu = cu_seqlens_cpu
        ctx.chunk_indices = chunk_indices
        ctx.save_for_backward(x, weight, bias, residual, initial_state)
        return causal_conv1d_fwd(
            x=x, weight=weight, bias=bias, residual=residual, initial_state=initial_state,
            output_final_state=output_final_state, activation=activation, cu_seqlens=cu_seqlens, cu_seqlens_cpu=cu_seqlens_cpu)

    @staticmethod
    def backward(ctx, dy, dht=None):
        x, weight, bias, residual, initial_state = ctx.saved_tensors
        dx, dw, db, dr, dh0 = causal_conv1d_bwd(
            x=x, dy=dy, dht=dht, weight=weight, bias=bias, residual=residual, initial_state=initial_state,
            activation=ctx.activation, cu_seqlens=ctx.cu_seqlens, cu_seqlens_cpu=ctx.cu_seqlens_cpu,
            chunk_indices=ctx.chunk_indices)
        if residual is not None and dr.dtype != residual.dtype:
            dr = dr.to(residual.dtype)
        return dx, dw, db, dr, dh0, None, None, None, None, None


@input_guard(no_guard_contiguous=['x'])
def causal_conv1d_update_states(
    x: torch.Tensor,
    state_len: int,
    initial_state: torch.Tensor | None = None,
    cu_seqlens: torch.Tensor | None = None,
) -> torch.Tensor:
    """The state ``[N, D, state_len]`` a prefill over ``x`` leaves behind (no output is computed)."""
    if state_len > MAX_KERNEL_SIZE:
        raise NotImplementedError(f'kernel sizes above {MAX_KERNEL_SIZE} are not supported (got {state_len})')
    if x.dim() == 2:
        if cu_seqlens is None:
            raise ValueError('x of shape [T, D] needs `cu_seqlens`')
        x = x.unsqueeze(0)
    x = _rows(x, x.shape[-1])
    _, final_state = _launch_fwd(x, None, None, None, initial_state, False, True, None, cu_seqlens, state_len)
    return final_state


@input_guard(no_guard_contiguous=['x'])
def causal_conv1d_update(
    x: torch.Tensor,
    cache: torch.Tensor,
    residual: torch.Tensor | None = None,
    weight: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    activation: str | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """One new token per sequence: ``x`` is ``[N, D]``, ``[1, N, D]`` or ``[N, 1, D]``; ``cache`` ``[N, D, W]`` is
    updated in place (shifted left by one, ``x`` appended) and returned."""
    forward_only('causal_conv1d_update', x, residual)
    if weight is None:
        raise ValueError('causal_conv1d_update needs a weight of shape [D, W]')
    dev = require_gpu(x)
    shape = x.shape
    D, W = weight.shape
    if W > MAX_KERNEL_SIZE:
        raise NotImplementedError(f'kernel sizes above {MAX_KERNEL_SIZE} are not supported (got {W})')
    if x.shape[-1] != D:
        x = x.reshape(x.shape[0], x.shape[1], -1)
    if x.dim() == 2:                                  # [N, D]
        rows = x
    elif x.dim() == 3 and x.shape[0] == 1:            # [1, N, D]: packed layout, one token per sequence
        rows = x[0]
    elif x.dim() == 3 and x.shape[1] == 1:            # [N, 1, D]
        rows = x[:, 0]
    else:
        raise ValueError(f'Unsupported input shape: {x.shape}')
    if rows.stride(-1) != 1:
        rows = rows.contiguous()
    N = rows.shape[0]
    if cache is not None:
        if tuple(cache.shape) != (N, D, W):
            raise ValueError(f'cache must be [{N}, {D}, {W}], got {tuple(cache.shape)}')
        if not cache.is_contiguous():
            raise ValueError('cache must be contiguous: it is updated in place')
    y = torch.empty(N, D, dtype=x.dtype, device=dev)
    if residual is not None:
        residual = residual.reshape(N, D).to(x.dtype).contiguous()
    if bias is not None and bias.dtype != weight.dtype:
        bias = bias.to(weight.dtype)
    with torch.cuda.device(dev):
        _lib.check(_lib.load().gdn_causal_conv1d_update(
            ptr(rows), ptr(cache), ptr(residual), ptr(weight), ptr(bias), ptr(y),
            N, D, W, rows.stride(0) if N > 1 else D, D,
            dtype_code(x.dtype), dtype_code(weight.dtype),
            dtype_code(cache.dtype) if cache is not None else _lib.DTYPE_F32,
            _activation_code(activation), current_stream_ptr(dev)))
    return y.view(shape), cache


@input_guard(no_guard_contiguous=['x'])
def causal_conv1d(
    x: torch.Tensor,
    weight: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    residual: torch.Tensor | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool | None = False,
    activation: str | None = None,
    backend: str | None = 'triton',
    cu_seqlens: torch.Tensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
    chunk_indices: torch.LongTensor | None = None,
    cp_context=None,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Causal 1D convolution over ``x [B, T, D]`` with ``weight [D, W]``; returns ``(y, final_state)``.
    Every value of ``backend`` the reference accepts (`triton`, `cuda`, `mix`) runs the same HIP kernels.  Differentiable
    in x, weight, bias, residual and initial_state."""
    if cp_context is not None:
        raise NotImplementedError('context parallelism (cp_context) spans several GPUs and is not supported')
    if backend not in ('triton', 'cuda', 'mix'):
        raise ValueError(f'Unsupported backend: {backend}')
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (x, weight, bias, residual, initial_state)):
        if weight is None:
            raise ValueError('causal_conv1d_fwd needs a weight of shape [D, W]')
        if weight.shape[1] > MAX_KERNEL_SIZE:
            raise NotImplementedError(f'kernel sizes above {MAX_KERNEL_SIZE} are not supported (got {weight.shape[1]})')
        return CausalConv1dFunction.apply(x, weight, bias, residual, initial_state, bool(output_final_state), activation,
                                          cu_seqlens, cu_seqlens_cpu, chunk_indices)
    return causal_conv1d_fwd(
        x=x, weight=weight, bias=bias, residual=residual, initial_state=initial_state,
        output_final_state=output_final_state, activation=activation,
        cu_seqlens=cu_seqlens, cu_seqlens_cpu=cu_seqlens_cpu, chunk_indices=chunk_indices)


class ShortConvolution(nn.Conv1d):
    """Depthwise causal convolution layer with the reference's parameters and call signature
    (fla/modules/conv/short_conv.py:24-250); the prefill form is differentiable, the one-token step is not."""

    def __init__(
        self,
        hidden_size: int,
        kernel_size: int,
        bias: bool = False,
        activation: str | None = 'silu',
        backend: str | None = 'triton',
        device: torch.device | None = None,
        dtype: torch.dtype | None = None,
        **kwargs,
    ):
        super().__init__(in_channels=hidden_size, out_channels=hidden_size, kernel_size=kernel_size,
                         groups=hidden_size, bias=bias, padding=kernel_size - 1, device=device, dtype=dtype)
        self.hidden_size = hidden_size
        self.activation = None
        if activation is not None:
            assert activation in ['silu', 'swish'], f'Activation `{activation}` not supported yet.'
            self.activation = activation
        if 'use_fast_conv1d' in kwargs:
            warnings.warn('The `use_fast_conv1d` parameter is deprecated and will be ignored. '
                          'Please use the `backend` parameter instead.')
        self.backend = os.environ.get('FLA_CONV_BACKEND', backend)
        if backend not in ['cuda', 'triton']:
            raise ValueError(f"Invalid backend: {backend}, must be one of ['cuda', 'triton']")

    def extra_repr(self):
        s = super().extra_repr()
        if self.activation is not None:
            s += f', activation={self.activation}'
        return s + f', backend={self.backend}'

    def forward(
        self,
        x: torch.Tensor,
        residual: torch.Tensor | None = None,
        mask: torch.Tensor | None = None,
        cache: torch.Tensor | None = None,
        output_final_state: bool = False,
        cu_seqlens: torch.LongTensor | None = None,
        chunk_indices: torch.LongTensor | None = None,
        **kwargs,
    ) -> tuple[torch.Tensor, torch.Tensor | None]:
        B, T, *_ = x.shape
        N = B if cu_seqlens is None else len(cu_seqlens) - 1
        if mask is not None:
            if cu_seqlens is not None:
                raise ValueError('`mask` and `cu_seqlens` cannot be provided at the same time')
            x = x.mul_(mask.unsqueeze(-1))
        if B * T == N:                                # decoding: one token per sequence, cache updated in place
            return self.step(x=x, residual=residual, cache=cache, output_final_state=output_final_state,
                             cu_seqlens=cu_seqlens)
        return causal_conv1d(
            x=x, weight=self.weight.squeeze(1), bias=self.bias, residual=residual, initial_state=cache,
            output_final_state=output_final_state, activation=self.activation, backend='triton',
            cu_seqlens=cu_seqlens, chunk_indices=chunk_indices, **kwargs)

    def step(
        self,
        x: torch.Tensor,
        residual: torch.Tensor | None,
        cache: torch.Tensor | None,
        output_final_state: bool = False,
        cu_seqlens: torch.LongTensor | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor | None]:
        B, _, D = x.shape
        W = self.kernel_size[0]
        N = B if cu_seqlens is None else len(cu_seqlens) - 1
        if cache is None:
            cache = x.new_zeros(N, D, W)
        y, cache = causal_conv1d_update(x=x, cache=cache, residual=residual, weight=self.weight.squeeze(1),
                                        bias=self.bias, activation=self.activation)
        return y, (cache if output_final_state else None)

    @property
    def state_size(self) -> int:
        return self.hidden_size * self.kernel_size
