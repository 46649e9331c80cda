"""Host-side helpers shared by the two operators: dtype codes, pointer extraction,
argument normalisation.  Nothing here computes on tensors beyond casts/copies."""
from __future__ import annotations

import torch

from fla_hip import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.DTYPE_BF16, torch.float16: _lib.DTYPE_F16, torch.float32: _lib.DTYPE_F32}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise NotImplementedError(f'dtype {dt} is not supported by the HIP kernels (bf16, fp16, fp32)') from None


def ptr(x: torch.Tensor | None) -> int | None:
    return None if x is None else x.data_ptr()


def require_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    if dev.type != 'cuda':
        raise RuntimeError(
            'fla_hip runs only on a ROCm GPU (tensors must live on a "cuda" device); '
            'there is no CPU implementation behind this operator.')
    for t in tensors:
        if t is not None and t.device != dev:
            raise ValueError(f'all tensors must be on {dev}, got {t.device}')
    return dev


def as_f32(x: torch.Tensor | None) -> torch.Tensor | None:
    if x is None:
        return None
    return x if x.dtype == torch.float32 else x.float()


def pad_last_two(x: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """Zero-pads the last two dims up to ``rows x cols``; the tensor itself when nothing is missing (``F.pad`` by zero
    would still copy it: a pool of states per decode step)."""
    r, c = rows - x.shape[-2], cols - x.shape[-1]
    return x if r == 0 and c == 0 else torch.nn.functional.pad(x, (0, c, 0, r))


def aligned16(x: torch.Tensor | None) -> torch.Tensor | None:
    """The kernels read states with 16-byte vector loads."""
    if x is None or x.data_ptr() % 16 == 0:
        return x
    return x.clone(memory_format=torch.contiguous_format)


def unify_qkv(q, k, v):
    """q, k, v must share one of bf16/fp16/fp32; mixed inputs are cast to q's dtype."""
    dt = q.dtype
    if dt not in _DTYPE_CODE:
        raise NotImplementedError(f'q dtype {dt} is not supported (bf16, fp16, fp32)')
    return q, k.to(dt), v.to(dt)


def unify_gate_beta(g, beta):
    """g and beta are passed to the kernels with one shared dtype code."""
    present = [x for x in (g, beta) if x is not None]
    if not present:
        return g, beta, _lib.DTYPE_F32
    dts = {x.dtype for x in present}
    if len(dts) == 1 and present[0].dtype in _DTYPE_CODE:
        return g, beta, _DTYPE_CODE[present[0].dtype]
    return as_f32(g), as_f32(beta), _lib.DTYPE_F32


def check_operand_shapes(q, k, v, g=None, beta=None, gk=None, gv=None, beta_per_column: bool = False) -> None:
    """The kernels index every operand from B, T, H, K of q and HV, V of v: anything of another shape would be read out
    of bounds, so it is refused here.  q, k ``[B,T,H,K]``; v ``[B,T,HV,V]``; g, beta ``[B,T,HV]`` (a trailing dimension of 1
    is let through; beta ``[B,T,HV,V]`` where the operator takes one per value column); gk ``[B,T,HV,K]``; gv ``[B,T,HV,V]``."""
    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError(f'q, k, v must be [B, T, heads, dim], got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}')
    if k.shape != q.shape:
        raise ValueError(f'q and k must have the same shape, got {tuple(q.shape)} and {tuple(k.shape)}')
    if v.shape[:2] != q.shape[:2]:
        raise ValueError(f'v must share batch and sequence length with q, got {tuple(v.shape)} and {tuple(q.shape)}')
    B, T, H, K = q.shape
    HV, V = v.shape[2], v.shape[3]
    if HV % H != 0:
        raise ValueError(f'num_v_heads (HV={HV}) must be divisible by num_heads (H={H})')

    def per_head(x, name, last=None):
        want = (B, T, HV) if last is None else (B, T, HV, last)
        ok = tuple(x.shape) == want or (last is None and tuple(x.shape) == (B, T, HV, 1))
        if not ok:
            raise ValueError(f'{name} must have shape {want}, got {tuple(x.shape)}')

    if g is not None:
        per_head(g, 'g')
    if beta is not None:
        if beta_per_column and beta.dim() == 4 and beta.shape[-1] != 1:
            per_head(beta, 'beta', V)
        else:
            per_head(beta, 'beta')
    if gk is not None:
        per_head(gk, 'gk', K)
    if gv is not None:
        per_head(gv, 'gv', V)


def current_stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def forward_only(what: str, *activations: torch.Tensor | None) -> None:
    """Operators without a backward refuse activations that require a gradient (in grad mode) instead of returning a
    result that silently carries none.  Parameters are not looked at: inference outside ``torch.no_grad()`` is fine."""
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in activations):
        raise NotImplementedError(f'{what} has no backward in fla_hip: run it under torch.no_grad() or on detached inputs')
