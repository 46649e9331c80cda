"""``fused_recurrent_comba`` with the signature of fla/ops/comba/fused_recurrent.py:225-335 (mind the order: q, k, p, v).
The token recurrence (predict with p on the undecayed state, decay, write k; fused_recurrent.py:85-105) runs on the
token kernel of the gated delta rule in its comba form, one call into libgdn_hip.so (``gdn_fused_recurrent_comba_fwd``):
fp32 arithmetic and an fp32 state whatever the inputs' dtype, as in the reference (:147), beta per head or per value
column (:68-71), grouped value heads, packed sequences."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import (
    pad_last_two,
    aligned16,
    as_f32,
    check_operand_shapes,
    current_stream_ptr,
    dtype_code,
    forward_only,
    ptr,
    require_gpu,
    unify_gate_beta,
    unify_qkv,
)
from fla_hip.ops.utils.index import check_cu_seqlens


def fused_recurrent_comba_fwd(q, k, p, v, g, beta, scale, initial_state, output_final_state,
                              use_qk_l2norm_in_kernel=False, cu_seqlens=None):
    """Returns ``(o [B,T,HV,V] in v's dtype, final_state [N,HV,K,V] fp32 or None)``."""
    dev = require_gpu(q, k, p, v, g)
    check_operand_shapes(q, k, v, g=g, beta=beta, beta_per_column=True)
    if p.shape != q.shape:
        raise ValueError(f'q, k and p must share one shape, got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(p.shape)}')
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > 256:
        raise NotImplementedError(f'the token kernel covers key head dims up to 256 (got K={K})')
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    q, k, v = unify_qkv(q, k, v)
    p = p.to(q.dtype)
    g, beta, gb_code = unify_gate_beta(g, beta)
    # the kernel moves 16-byte pieces of state rows: head dims that are not multiples of 4 are zero-padded
    KP, VP = (K + 3) // 4 * 4, (V + 3) // 4 * 4
    flags = _lib.FLAG_QK_L2NORM if use_qk_l2norm_in_kernel else 0
    if beta is not None and beta.ndim == v.ndim:
        flags |= _lib.FLAG_BETA_VECTOR
    if (KP, VP) != (K, V):
        q, k, p, v = F.pad(q, (0, KP - K)), F.pad(k, (0, KP - K)), F.pad(p, (0, KP - K)), F.pad(v, (0, VP - V))
        if flags & _lib.FLAG_BETA_VECTOR:
            beta = F.pad(beta, (0, VP - V))
    q, k, p, v, g = (x.contiguous() for x in (q, k, p, v, g))
    beta = None if beta is None else beta.contiguous()
    h0 = None
    if initial_state is not None:
        if tuple(initial_state.shape) != (N, HV, K, V):
            raise ValueError(f'initial_state must have shape {(N, HV, K, V)}, got {tuple(initial_state.shape)}')
        h0 = aligned16(pad_last_two(as_f32(initial_state), KP, VP).contiguous())
    if cu_seqlens is not None:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            cu_seqlens = cu_seqlens.long()
        cu_seqlens = cu_seqlens.to(dev)
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        check_cu_seqlens(cu_seqlens, T)
    o = torch.empty_like(v)
    ht = torch.empty(N, HV, KP, VP, dtype=torch.float32, device=dev) if output_final_state else None
    _lib.check(_lib.load().gdn_fused_recurrent_comba_fwd(
        ptr(q), ptr(k), ptr(p), ptr(v), ptr(g), ptr(beta), ptr(h0), ptr(ht), ptr(o), ptr(cu_seqlens),
        B, T, H, HV, KP, VP, N, float(scale), dtype_code(q.dtype), gb_code, flags, current_stream_ptr(dev)))
    if (KP, VP) != (K, V):
        o = o[..., :V].contiguous()
        if ht is not None:
            ht = ht[..., :K, :V].contiguous()
    return o, ht


@torch.compiler.disable
def fused_recurrent_comba(
    q: torch.Tensor,
    k: torch.Tensor,
    p: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
):
    r"""Args as ``chunk_comba`` (``v``: ``[B, T, HV, V]``, grouped value heads allowed), in the reference's order
    ``q, k, p, v, g, beta``; beta ``[B, T, HV]`` or one per value column ``[B, T, HV, V]`` (ones when ``None``).
    Forward only, as in the reference (fla/ops/comba/fused_recurrent.py:217-222).

    Returns:
        ``(o [B, T, HV, V] in v's dtype, final_state [N, HV, K, V] fp32 or None)``.
    """
    if p is None:
        p = k
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.'
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    forward_only('fused_recurrent_comba', q, k, p, v, g, beta, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return fused_recurrent_comba_fwd(q, k, p, v, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel,
                                     cu_seqlens)
