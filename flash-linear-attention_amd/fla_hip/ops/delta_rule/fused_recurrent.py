"""``fused_recurrent_delta_rule``: the token recurrence of the delta rule without gates, with the signature of
fla/ops/delta_rule/fused_recurrent.py:443-532.  Forward: the gated kernel with g absent.  Backward (when an input
requires a gradient): ``gdn_fused_recurrent_delta_bwd``, one HIP kernel in place of the reference's
``fused_recurrent_delta_rule_bwd`` (:313-385), inside an autograd function of the reference's shape (:388-441)."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import aligned16, as_f32, current_stream_ptr, dtype_code, pad_last_two, ptr, require_gpu
from fla_hip.ops.gated_delta_rule.fused_recurrent import fused_recurrent_gated_delta_rule_fwd
from fla_hip.ops.utils.index import check_cu_seqlens, cu_bounds


def _pad_last(x: torch.Tensor, size: int) -> torch.Tensor:
    return x if x.shape[-1] == size else F.pad(x, (0, size - x.shape[-1]))


def fused_recurrent_delta_rule_bwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor | None,
    dht: torch.Tensor | None,
    do: torch.Tensor,
    scale: float,
    initial_state: torch.Tensor | None,
    cu_seqlens: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor | None, torch.Tensor | None]:
    """q, k ``[B,T,H,K]`` (as the recurrence uses them: after the l2 normalisation, if any), v, do ``[B,T,H,V]``,
    beta ``[B,T,H]`` or ``[B,T,H,V]`` or None.  Returns fp32 ``(dq, dk, dv, dbeta, dh0)`` (dbeta None without beta,
    dh0 None without ``initial_state``).  The kernel takes K in multiples of 16 and V in multiples of its value
    block: other head dims are zero-padded here."""
    dev = require_gpu(q, k, v, do)
    B, T, H, K = k.shape
    V = v.shape[-1]
    if K > 256:
        raise NotImplementedError(f'the backward kernel covers key head dims up to 256 (got K={K})')
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    lib = _lib.load()
    KP = (K + 15) // 16 * 16
    VB = lib.gdn_fused_recurrent_delta_bwd_value_block(KP)
    VP = (V + VB - 1) // VB * VB
    NVB = VP // VB
    work = q.dtype if q.dtype in (torch.bfloat16, torch.float16, torch.float32) else torch.float32
    qw, kw = (aligned16(_pad_last(x.to(work), KP).contiguous()) for x in (q, k))
    vw, dow = (aligned16(_pad_last(x.to(work), VP).contiguous()) for x in (v, do))
    flags = 0
    bw = None
    if beta is not None:
        bw = as_f32(beta)
        if beta.ndim == v.ndim:
            flags |= _lib.FLAG_BETA_VECTOR
            bw = _pad_last(bw, VP)
        bw = bw.contiguous()

    def state_in(s):
        if s is None:
            return None
        if tuple(s.shape) != (N, H, K, V):
            raise ValueError(f'initial_state and dht must have shape {(N, H, K, V)}, got {tuple(s.shape)}')
        return aligned16(pad_last_two(as_f32(s), KP, VP).contiguous())
    h0, dhtw = state_in(initial_state), state_in(dht)

    # tokens of a packed tensor outside every sequence are never written: they get zero gradients
    alloc = torch.empty
    if cu_seqlens is not None:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            cu_seqlens = cu_seqlens.long()
        cu_seqlens = cu_seqlens.to(dev)
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        check_cu_seqlens(cu_seqlens, T)
        first, last = cu_bounds(cu_seqlens)
        if first != 0 or last != T:
            alloc = torch.zeros
    f32 = dict(dtype=torch.float32, device=dev)
    dq_part, dk_part = alloc(NVB, B, T, H, KP, **f32), alloc(NVB, B, T, H, KP, **f32)
    dv = alloc(B, T, H, VP, **f32)
    db = alloc(B, T, H, VP, **f32) if flags & _lib.FLAG_BETA_VECTOR else alloc(NVB, B, T, H, **f32)
    dh0 = torch.empty(N, H, KP, VP, **f32) if initial_state is not None else None
    u = torch.empty(B, T, H, VP, **f32)
    _lib.check(lib.gdn_fused_recurrent_delta_bwd(
        ptr(qw), ptr(kw), ptr(vw), ptr(bw), ptr(dow), ptr(h0), ptr(dhtw),
        ptr(dq_part), ptr(dk_part), ptr(dv), ptr(db), ptr(dh0), ptr(u), ptr(cu_seqlens),
        B, T, H, KP, VP, N, float(scale), dtype_code(work), _lib.DTYPE_F32, flags, current_stream_ptr(dev)))
    dq, dk = dq_part.sum(0)[..., :K], dk_part.sum(0)[..., :K]
    dbeta = None
    if beta is not None:
        dbeta = db[..., :V] if flags & _lib.FLAG_BETA_VECTOR else db.sum(0)
    if dh0 is not None:
        dh0 = dh0[..., :K, :V].contiguous()
    return dq, dk, dv[..., :V], dbeta, dh0


def _l2norm(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Rows divided by sqrt(sum x^2 + 1e-6) in fp32, and that factor (fla/modules/l2norm.py: eps 1e-6)."""
    xf = x.float()
    rstd = torch.rsqrt(xf.square().sum(-1, keepdim=True) + 1e-6)
    return xf * rstd, rstd


class FusedRecurrentDeltaRuleFunction(torch.autograd.Function):
    """Forward through the token-recurrence kernel, backward through ``gdn_fused_recurrent_delta_bwd``.  Nothing is
    kept from the forward call but its inputs."""

    @staticmethod
    def forward(ctx, q, k, v, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel, cu_seqlens):
        o, ht = fused_recurrent_gated_delta_rule_fwd(
            q, k, v, beta=beta, scale=scale, initial_state=initial_state, output_final_state=output_final_state,
            use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, cu_seqlens=cu_seqlens)
        ctx.save_for_backward(q, k, v, beta, initial_state, cu_seqlens)
        ctx.opts = (scale, use_qk_l2norm_in_kernel)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        q, k, v, beta, h0, cu_seqlens = ctx.saved_tensors
        scale, l2 = ctx.opts
        qn, kn, q_rstd, k_rstd = q, k, None, None
        if l2:
            # the rows the recurrence saw, and the way back through the normalisation: elementwise work around the call
            (qn, q_rstd), (kn, k_rstd) = _l2norm(q), _l2norm(k)
        dq, dk, dv, db, dh0 = fused_recurrent_delta_rule_bwd(qn, kn, v, beta, dht, do.contiguous(), scale, h0, cu_seqlens)
        if l2:
            dq = (dq - qn * (qn * dq).sum(-1, keepdim=True)) * q_rstd
            dk = (dk - kn * (kn * dk).sum(-1, keepdim=True)) * k_rstd
        return (dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), None if beta is None else db.to(beta.dtype), None,
                None if h0 is None or not ctx.needs_input_grad[5] else dh0.to(h0.dtype), None, None, None)


@torch.compiler.disable
def fused_recurrent_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    r"""q, k ``[B, T, H, K]``, v ``[B, T, H, V]``, beta ``[B, T, H]`` or ``[B, T, H, V]`` (ones when omitted).
    Returns ``(o, final_state [N, H, K, V] fp32 or None)``; differentiable in q, k, v, beta and ``initial_state``."""
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.'
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    if scale is None:
        scale = k.shape[-1] ** -0.5
    else:
        assert scale > 0, 'scale must be positive'
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (q, k, v, beta, initial_state)):
        if v.shape[2] != k.shape[2]:
            raise NotImplementedError('the backward of fused_recurrent_delta_rule takes as many value heads as key heads')
        return FusedRecurrentDeltaRuleFunction.apply(q, k, v, beta, scale, initial_state, output_final_state,
                                                     use_qk_l2norm_in_kernel, cu_seqlens)
    return fused_recurrent_gated_delta_rule_fwd(
        q, k, v, beta=beta, scale=scale, initial_state=initial_state, output_final_state=output_final_state,
        use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, cu_seqlens=cu_seqlens)
