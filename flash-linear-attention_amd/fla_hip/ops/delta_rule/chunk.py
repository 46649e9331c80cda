"""``chunk_delta_rule``: the delta rule without gates (DeltaNet), with the signature,
validation and error types of fla/ops/delta_rule/chunk.py:223-349.  It is the gated operator with
g = 0 (the reference runs the same state and output kernels with ``g=None``,
fla/ops/delta_rule/chunk.py:39-62), so it runs on the same HIP kernels: the library takes
``g = NULL`` and skips nothing but the gate load.  Differentiable like the gated operator (backward through
``gdn_chunk_bwd`` with ``g = NULL``; the reference's own backward is fla/ops/delta_rule/chunk.py:65-140)."""
from __future__ import annotations

import torch

from fla_hip.ops.gated_delta_rule.chunk import chunk_gated_delta_rule_fwd


@torch.compiler.disable
def chunk_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor,
    scale: float | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
    **kwargs,
):
    r"""
    Args:
        q, k: ``[B, T, H, K]``; v: ``[B, T, H, V]``; beta: ``[B, T, H]``; bf16 or fp16.
        scale: defaults to ``K ** -0.5``.
        initial_state: ``[N, H, K, V]``; output_final_state: also return the fp32 final state.
        use_qk_l2norm_in_kernel: L2-normalise q and k per head first.
        cu_seqlens: ``[N + 1]`` boundaries of packed sequences (then ``B == 1``); ``cu_seqlens_cpu``
            an optional host copy that avoids a device sync.

    Returns:
        ``(o [B, T, H, V] in q's dtype, final_state or None)``.
    """
    assert q.dtype == k.dtype == v.dtype
    assert q.dtype != torch.float32, 'chunk_delta_rule does not support float32. Please use bfloat16.'
    assert len(beta.shape) == 3, 'beta must be of shape (batch size, seq len, num of head).'
    if 'head_first' in kwargs:
        raise DeprecationWarning('head_first has been removed. Inputs must be in `[B, T, H, ...]` format.')
    chunk_size = kwargs.pop('chunk_size', 64)
    if chunk_size not in (16, 32, 64):
        raise ValueError(f'`chunk_size` must be 16, 32, or 64, got {chunk_size}.')
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`. '
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    scale = k.shape[-1] ** -0.5 if scale is None else scale
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (q, k, v, beta, initial_state)):
        from fla_hip.ops.gated_delta_rule.chunk_bwd import ChunkGatedDeltaRuleFunction
        return ChunkGatedDeltaRuleFunction.apply(
            q, k, v, None, beta, scale, initial_state, output_final_state, False, cu_seqlens, cu_seqlens_cpu, None,
            use_qk_l2norm_in_kernel, False, None, None, False, False, chunk_size)
    return chunk_gated_delta_rule_fwd(
        q, k, v, None, beta, scale, initial_state, output_final_state, False,
        cu_seqlens, cu_seqlens_cpu, None, chunk_size, None, None, use_qk_l2norm_in_kernel, False, False)
